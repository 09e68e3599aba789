// The gated delta rule: a mixer whose memory is one matrix per head instead of a cache of keys and values.
//
// Per value head h (reading key/query head h / (H / G)) and token, with S of size [D keys, Dv values] in 32-bit:
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// so the read-out sees the token's own write. q, k and v come out of a short causal convolution over time per
// channel (taps weights, the last one the current token's, zeros before a sequence's start) followed by silu; q and
// k are then scaled to unit length per head, x / sqrt(sum x^2 + unit_eps), and q by q_scale. The decay is
// g = exp(-exp(A_log[h]) softplus(a + dt_bias[h])), the write strength beta = sigmoid(b); a and b are two more
// columns per head of the same projection. Everything here is computed in 32-bit, with accurate exp and log.
//
// A sequence's state, one row of a [slots][state_stride] float array:
//   S in tiles of 16 value columns, [H][ceil(Dv / 16)][D][16] (a wave's share of S is consecutive memory),
//   then the convolution's last taps - 1 inputs of each of the C = 2 G D + H Dv channels, [C][taps - 1], oldest first.
// The tokens of a step are packed, sequence after sequence (cu_seqlens); each sequence is walked token by token from
// the state that earlier steps left, so a result does not depend on how the tokens were cut into steps.
//
// Two entry points: delta_prep (convolution, silu, unit length, decay and strength; then the convolution's new
// state) and delta_recurrence (the rule itself, then each head's read-out divided by its root mean square, times a
// weight shared by the heads, times silu of a gate).
#include "common.h"

__device__ __forceinline__ float dr_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float dr_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

struct DeltaShape {
  int H, G, D, Dv, taps;
  int ldp;            // floats a row of the projection
  int off_q, off_k, off_v, off_b, off_a;   // first column of each part in a row of the projection
  long state_stride;  // floats a slot
  long conv_off;      // where the convolution's inputs start in a slot's state
};

// grid (T, 2 G + H + 1): a q head, a k head, a v head, or the token's decays and strengths. One wave.
// one_each: every sequence of the step brings exactly one token (a decode step); the held inputs then move on here.
__global__ __launch_bounds__(64) void delta_prep_kernel(
    const float* __restrict__ proj, const float* __restrict__ conv_w, const float* __restrict__ A_log,
    const float* __restrict__ dt_bias, float* __restrict__ state, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_of_token, const int* __restrict__ slot_ids, float* __restrict__ act,
    float* __restrict__ gates, DeltaShape s, float unit_eps, float q_scale, int one_each) {
  const int t = blockIdx.x, u = blockIdx.y, lane = threadIdx.x;
  const int C = 2 * s.G * s.D + s.H * s.Dv;
  const float* row = proj + (long)t * s.ldp;
  if (u == 2 * s.G + s.H) {
    for (int h = lane; h < s.H; h += 64) {
      const float sp = dr_softplus(row[s.off_a + h] + dt_bias[h]);
      gates[(long)t * 2 * s.H + h] = expf(-expf(A_log[h]) * sp);
      gates[(long)t * 2 * s.H + s.H + h] = dr_sigmoid(row[s.off_b + h]);
    }
    return;
  }
  const int b = seq_of_token[t];
  const int first = cu_seqlens[b], i = t - first;
  float* held = state + (long)slot_ids[b] * s.state_stride + s.conv_off;
  // the unit's channels: c0 .. c0 + n of the C convolved channels, which are columns col0 .. of the projection
  int c0, col0, n;
  if (u < s.G) { c0 = u * s.D; col0 = s.off_q + u * s.D; n = s.D; }
  else if (u < 2 * s.G) { c0 = s.G * s.D + (u - s.G) * s.D; col0 = s.off_k + (u - s.G) * s.D; n = s.D; }
  else { c0 = 2 * s.G * s.D + (u - 2 * s.G) * s.Dv; col0 = s.off_v + (u - 2 * s.G) * s.Dv; n = s.Dv; }
  const bool unit = u < 2 * s.G;
  float ss = 0.f;
  for (int e = lane; e < n; e += 64) {
    const int c = c0 + e;
    float y = 0.f;
    for (int r = 0; r < s.taps; ++r) {
      const int src = i - (s.taps - 1 - r);
      const float x = src >= 0 ? proj[(long)(first + src) * s.ldp + col0 + e] : held[(long)c * (s.taps - 1) + src + s.taps - 1];
      y = fmaf(conv_w[(long)c * s.taps + r], x, y);
    }
    y = y * dr_sigmoid(y);
    ss = fmaf(y, y, ss);
    act[(long)t * C + c] = y;
    if (one_each && s.taps > 1) {
      // every sequence brings one token: this lane is the only reader of the channel's held inputs, and moves them on
      float* hc = held + (long)c * (s.taps - 1);
      for (int jj = 0; jj + 2 < s.taps; ++jj) hc[jj] = hc[jj + 1];
      hc[s.taps - 2] = proj[(long)t * s.ldp + col0 + e];
    }
  }
  if (!unit) return;
  ss = wave_sum(ss);
  const float f = (u < s.G ? q_scale : 1.0f) / sqrtf(ss + unit_eps);
  for (int e = lane; e < n; e += 64) act[(long)t * C + c0 + e] *= f;   // (the lane's own stores of above)
}

// grid (B, ceil(C / 256)): a thread moves one channel's held inputs on by the sequence's new tokens, oldest first,
// so that no place is written before it has been read.
__global__ __launch_bounds__(256) void delta_conv_state_kernel(const float* __restrict__ proj, float* __restrict__ state,
                                                               const int* __restrict__ cu_seqlens,
                                                               const int* __restrict__ slot_ids, DeltaShape s) {
  const int b = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  const int GD = s.G * s.D, C = 2 * GD + s.H * s.Dv;
  if (c >= C) return;
  const int first = cu_seqlens[b], n = cu_seqlens[b + 1] - first;
  if (n <= 0) return;
  const int col = c < GD ? s.off_q + c : c < 2 * GD ? s.off_k + (c - GD) : s.off_v + (c - 2 * GD);
  float* held = state + (long)slot_ids[b] * s.state_stride + s.conv_off + (long)c * (s.taps - 1);
  for (int j = 0; j < s.taps - 1; ++j) {
    const int src = n - (s.taps - 1) + j;
    held[j] = src >= 0 ? proj[(long)(first + src) * s.ldp + col] : held[j + n];
  }
}

// The rule itself and the read-out's norm. grid (H, B, blocks a head: 1 unless the launcher deals a prompt's head out), a block of ceil(Dv / 16) waves: wave w owns the 16 value
// columns 16 w .. of head h's matrix, lane (r, c) of it the rows r, r + 4, ... of column c (RPL rows a lane), so a
// token costs a lane RPL multiply-adds for each of S^T k, the update and S^T q, and the sums over the four lanes of
// a column are two lane swaps each (no trip through shared memory). The tokens' operands (k, q, v, decay,
// strength) come in chunks of DR_CHUNK tokens through shared memory, the next chunk's loads on their way while
// the current chunk is worked on: what a token waits for is its own chain of multiply-adds, not memory.
// After the last token the block divides each of its tokens' read-outs (which it wrote to `o` itself) by their
// root mean square over the head and applies the weight and the gate: y = o / rms * w * silu(gate).
#define DR_CHUNK 16   // the most tokens a chunk; the launcher takes fewer where keys and values are long
#define DR_NLD 8       // loads a thread has on their way for the next chunk

__device__ __forceinline__ float dr_sum4(float p) {   // the sum over lanes l, l ^ 16, l ^ 32, l ^ 48
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(p), __float_as_uint(p), false, false);
  p = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(p), __float_as_uint(p), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// RG: the lanes a column's rows are dealt out to, 4 (16 columns a wave) or 8 (8 columns a wave: twice the waves with
// half the work per token each, which is what a prompt's long chains of tokens want; the state lies the same).
template <int RG>
__device__ __forceinline__ float dr_sum_rows(float p) {
  if (RG == 8)    // lane l ^ 8 is 8 places round the row of 16
    p += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(p), 0x128, 0xf, 0xf, false));
  return dr_sum4(p);
}

template <int RPL, typename TO, int MAXT, int RG>
__global__ __launch_bounds__(MAXT) void delta_recurrence_kernel(
    const float* __restrict__ act, const float* __restrict__ gates, float* __restrict__ state,
    const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids, float* __restrict__ o,
    const float* __restrict__ proj, int ldp, int off_gate, const float* __restrict__ norm_w, TO* __restrict__ y,
    float eps, DeltaShape s, int chunk, int norm_here, int own_waves) {
  extern __shared__ __attribute__((aligned(16))) float dr_lds[];   // two buffers of chunk * per_token floats
  typedef float f4 __attribute__((ext_vector_type(4)));
  const int h = blockIdx.x, b = blockIdx.y;
  constexpr int COLS = 64 / RG;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane / COLS, c = lane % COLS;
  const int D = s.D, H = s.H, Dv = s.Dv;
  // (a head's columns may be dealt out to several blocks, blockIdx.z: own_waves waves of columns each)
  const int j = ((int)blockIdx.z * own_waves + wave) * COLS + c;
  const bool valid = wave < own_waves && j < Dv;
  const int C = 2 * s.G * D + H * Dv;
  const int kvh = h / (H / s.G);
  const int first = cu_seqlens[b], last = cu_seqlens[b + 1];
  if (last <= first) return;
  const int CT = (Dv + 15) / 16;
  const bool owner = wave < own_waves && j < CT * 16;     // (a block may have more waves than columns to own: they only help to load)
  // the lane's column in the state's tiles of 16 columns: row i of it at [16 i]
  float* tile = state + (long)slot_ids[b] * s.state_stride + ((long)(h * CT + (owner ? j / 16 : 0)) * D) * 16 + (j & 15);
  float S[RPL];
#pragma unroll
  for (int ii = 0; ii < RPL; ++ii) {
    const int i = r + RG * ii;
    S[ii] = (owner && i < D) ? tile[(long)i * 16] : 0.f;
  }
  // A token's operands in a chunk's buffer: q | k | v [Dv] | decay, strength, where q and k lie as the lanes read
  // them: row r + RG ii at [r][ii], RPL places a lane (rows beyond D stay zero), so a lane's share is 16-byte reads.
  const int per_src = 2 * D + Dv + 2;                           // what a token brings
  constexpr int VEC = RG * RPL;                                 // places of q, and of k
  const int per_token = 2 * VEC + ((Dv + 2 + 3) & ~3);          // what it takes in the buffer
  const int n_src = chunk * per_src;
  const long q_at = (long)kvh * D, k_at = (long)s.G * D + (long)kvh * D, v_at = 2L * s.G * D + (long)h * Dv;
  const int threads = blockDim.x;
  for (int e = tid; e < 2 * chunk * per_token; e += threads) dr_lds[e] = 0.f;
  __syncthreads();
  float held[DR_NLD];
  auto ask = [&](int t0) {
#pragma unroll
    for (int n = 0; n < DR_NLD; ++n) {
      const int e = tid + n * threads;
      const int tt = e / per_src, f = e - tt * per_src, t = t0 + tt;
      const float* p = act;
      if (e < n_src && t < last) {
        if (f < D) p = act + (long)t * C + q_at + f;
        else if (f < 2 * D) p = act + (long)t * C + k_at + (f - D);
        else if (f < 2 * D + Dv) p = act + (long)t * C + v_at + (f - 2 * D);
        else p = gates + (long)t * 2 * H + (long)(f - 2 * D - Dv) * H + h;
      }
      held[n] = *p;
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int n = 0; n < DR_NLD; ++n) {
      const int e = tid + n * threads;
      if (e < n_src) {
        const int tt = e / per_src, f = e - tt * per_src;
        int at;
        if (f < 2 * D) {
          const int which = f >= D, i = f - which * D;
          at = which * VEC + (i % RG) * RPL + i / RG;
        } else {
          at = 2 * VEC + (f - 2 * D);
        }
        dr_lds[(buf * chunk + tt) * per_token + at] = held[n];
      }
    }
  };
  ask(first);
  put(0);
  __syncthreads();
  int buf = 0;
  for (int t0 = first; t0 < last; t0 += chunk) {
    const bool more = t0 + chunk < last;
    if (more) ask(t0 + chunk);
    const int n_here = min(chunk, last - t0);
    // two tokens' operands in registers in turn: the next token's reads from shared memory are on their way while
    // the current token's chain of multiply-adds runs
    struct Operands { float k[RPL], q[RPL], v, g, beta; };
    auto fetch = [&](Operands& x, int tt) {
      const float* op = dr_lds + (buf * chunk + tt) * per_token;
#pragma unroll
      for (int ii = 0; ii < RPL; ii += 4) {
        const f4 q4 = *(const f4*)(op + r * RPL + ii), k4 = *(const f4*)(op + VEC + r * RPL + ii);
#pragma unroll
        for (int e = 0; e < 4; ++e) { x.q[ii + e] = q4[e]; x.k[ii + e] = k4[e]; }
      }
      x.g = op[2 * VEC + Dv];
      x.beta = op[2 * VEC + Dv + 1];
      x.v = valid ? op[2 * VEC + j] : 0.f;
    };
    auto work = [&](const Operands& x, int tt) {
      float p4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < RPL; ++ii) {
        S[ii] *= x.g;
        p4[ii & 3] = fmaf(S[ii], x.k[ii], p4[ii & 3]);
      }
      const float part = dr_sum_rows<RG>((p4[0] + p4[1]) + (p4[2] + p4[3]));
      const float uu = x.beta * (x.v - part);
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < RPL; ++ii) {
        S[ii] = fmaf(x.k[ii], uu, S[ii]);
        o4[ii & 3] = fmaf(S[ii], x.q[ii], o4[ii & 3]);
      }
      const float read = dr_sum_rows<RG>((o4[0] + o4[1]) + (o4[2] + o4[3]));
      if (r == 0 && valid) o[(long)(t0 + tt) * H * Dv + (long)h * Dv + j] = read;
    };
    if constexpr (RPL <= 24 && MAXT <= 512) {
      // (pairs of tokens without a branch between them, so that the end of one token's work, which nothing waits
      // for, can be scheduled into the start of the next one's)
      Operands xa, xb;
      fetch(xa, 0);
      int tt = 0;
      for (; tt + 2 <= n_here; tt += 2) {
        fetch(xb, tt + 1);
        work(xa, tt);
        fetch(xa, min(tt + 2, n_here - 1));
        work(xb, tt + 1);
      }
      if (tt < n_here) work(xa, tt);
    } else {                              // (long keys, or a block of sixteen waves: two tokens' operands beside the matrix do not fit the registers)
      Operands xa;
      for (int tt = 0; tt < n_here; ++tt) {
        fetch(xa, tt);
        work(xa, tt);
      }
    }
    if (more) put(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }
#pragma unroll
  for (int ii = 0; ii < RPL; ++ii) {
    const int i = r + RG * ii;
    if (owner && i < D) tile[(long)i * 16] = S[ii];
  }
  // (steps of many tokens a sequence: a launch of its own, with a wave to every token and head, normalises them)
  if (!norm_here) return;
  // the read-outs of this head are all this block's own stores: made visible to its other waves, then normalised
  __threadfence_block();
  __syncthreads();
  const int n_waves = threads >> 6;
  for (int t = first + wave; t < last; t += n_waves) {
    const float* orow = o + ((long)t * H + h) * Dv;
    const float* grow = proj + (long)t * ldp + off_gate + (long)h * Dv;
    float ss = 0.f;
    for (int e = lane; e < Dv; e += 64) {
      const float x = orow[e];
      ss = fmaf(x, x, ss);
    }
    ss = wave_sum(ss);
    const float f = 1.0f / sqrtf(ss / (float)Dv + eps);
    TO* dst = y + ((long)t * H + h) * Dv;
    for (int e = lane; e < Dv; e += 64) {
      const float z = grow[e];
      dst[e] = from_f32<TO>(orow[e] * f * norm_w[e] * (z * dr_sigmoid(z)));
    }
  }
}

// grid (T, H), one wave: y[t, h, :] = o / sqrt(mean(o^2) + eps) * w * silu(gate[t, h, :])
template <typename TO>
__global__ __launch_bounds__(64) void delta_gated_norm_kernel(const float* __restrict__ o, const float* __restrict__ proj,
                                                              int ldp, int off_gate, const float* __restrict__ w,
                                                              TO* __restrict__ y, int H, int Dv, float eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + ((long)t * H + h) * Dv;
  const float* grow = proj + (long)t * ldp + off_gate + (long)h * Dv;
  float ss = 0.f;
  for (int e = lane; e < Dv; e += 64) ss = fmaf(orow[e], orow[e], ss);
  ss = wave_sum(ss);
  const float f = 1.0f / sqrtf(ss / (float)Dv + eps);
  TO* dst = y + ((long)t * H + h) * Dv;
  for (int e = lane; e < Dv; e += 64) {
    const float z = grow[e];
    dst[e] = from_f32<TO>(orow[e] * f * w[e] * (z * dr_sigmoid(z)));
  }
}

static int delta_shape(DeltaShape& s, int H, int G, int D, int Dv, int taps, int ldp, int off_q, int off_k, int off_v,
                       int off_b, int off_a, long state_stride) {
  GL3_REQUIRE(H > 0 && G > 0 && H % G == 0 && D > 0 && D <= 256 && Dv > 0 && taps >= 1 && taps <= 64,
              "delta rule: %d heads over %d key heads of %d, values of %d, %d taps", H, G, D, Dv, taps);
  const long CT = (Dv + 15) / 16, C = 2L * G * D + (long)H * Dv;
  s = DeltaShape{H, G, D, Dv, taps, ldp, off_q, off_k, off_v, off_b, off_a, state_stride, (long)H * CT * D * 16};
  GL3_REQUIRE(state_stride >= s.conv_off + C * (taps - 1), "delta rule: a slot's state of %ld floats is too small",
              state_stride);
  const int ends[5] = {off_q + G * D, off_k + G * D, off_v + H * Dv, off_b + H, off_a + H};
  for (int i = 0; i < 5; ++i) GL3_REQUIRE(ends[i] <= ldp, "delta rule: the projection's rows of %d are too short", ldp);
  GL3_REQUIRE(off_q >= 0 && off_k >= 0 && off_v >= 0 && off_b >= 0 && off_a >= 0, "delta rule: a negative column");
  return 0;
}

extern "C" long gl3_delta_state_floats(int H, int G, int D, int Dv, int taps) {
  return (long)H * ((Dv + 15) / 16) * D * 16 + (2L * G * D + (long)H * Dv) * (taps - 1);
}

// proj [T][ldp] float: the projection of the step's tokens. conv_w [C][taps], A_log [H], dt_bias [H] float.
// state [slots][state_stride] float. act [T][C] and gates [T][2 H] float are written; then the held inputs move on
// (one_each: the caller vouches that every sequence brings exactly one token, and they move on in the same launch).
extern "C" int gl3_delta_prep(const float* proj, const float* conv_w, const float* A_log, const float* dt_bias,
                              float* state, const int* cu_seqlens, const int* seq_of_token, const int* slot_ids,
                              float* act, float* gates, int T, int B, int H, int G, int D, int Dv, int taps, int ldp,
                              int off_q, int off_k, int off_v, int off_b, int off_a, long state_stride, float unit_eps,
                              float q_scale, int one_each, hipStream_t stream) {
  if (T == 0 || B == 0) return 0;
  GL3_REQUIRE(proj && conv_w && A_log && dt_bias && state && cu_seqlens && seq_of_token && slot_ids && act && gates &&
                  T > 0 && B > 0, "gl3_delta_prep: bad arguments");
  DeltaShape s;
  if (delta_shape(s, H, G, D, Dv, taps, ldp, off_q, off_k, off_v, off_b, off_a, state_stride)) return -1;
  GL3_REQUIRE(2 * G + H + 1 <= 65535 && B <= 65535, "gl3_delta_prep: too many heads or sequences for the grid");
  delta_prep_kernel<<<dim3(T, 2 * G + H + 1), dim3(64), 0, stream>>>(proj, conv_w, A_log, dt_bias, state, cu_seqlens,
                                                                     seq_of_token, slot_ids, act, gates, s, unit_eps, q_scale, one_each);
  GL3_LAUNCH_CHECK();
  GL3_REQUIRE(!one_each || T == B, "gl3_delta_prep: %d tokens of %d sequences are not one each", T, B);
  if (taps > 1 && !one_each) {
    const int C = 2 * G * D + H * Dv;
    delta_conv_state_kernel<<<dim3(B, (C + 255) / 256), dim3(256), 0, stream>>>(proj, state, cu_seqlens, slot_ids, s);
    GL3_LAUNCH_CHECK();
  }
  return 0;
}

// act [T][C], gates [T][2 H] as gl3_delta_prep left them. o [T][H Dv] float receives the raw read-outs (scratch);
// y [T][H Dv] (float or bfloat16) the read-outs divided by their root mean square over each head, times norm_w [Dv]
// (float), times silu of the gate, whose H Dv columns start at off_gate of proj [T][ldp] (float).
extern "C" int gl3_delta_recurrence(const float* act, const float* gates, float* state, const int* cu_seqlens,
                                    const int* slot_ids, float* o, const float* proj, int ldp, int off_gate,
                                    const float* norm_w, void* y, int y_dtype, float eps, int T, int B, int H, int G, int D,
                                    int Dv, int taps, long state_stride, hipStream_t stream) {
  if (B == 0 || T == 0) return 0;
  GL3_REQUIRE(act && gates && state && cu_seqlens && slot_ids && o && proj && norm_w && y && B > 0,
              "gl3_delta_recurrence: bad arguments");
  DeltaShape s;
  if (delta_shape(s, H, G, D, Dv, taps, 1 << 30, 0, 0, 0, 0, 0, state_stride)) return -1;
  GL3_REQUIRE(H <= 65535 && B <= 65535, "gl3_delta_recurrence: too many heads or sequences for the grid");
  GL3_REQUIRE(Dv <= 256, "gl3_delta_recurrence: values of %d elements: a block holds up to 256 columns", Dv);
  GL3_REQUIRE(off_gate >= 0 && off_gate + H * Dv <= ldp, "gl3_delta_recurrence: the gate's columns %d .. of rows of %d", off_gate, ldp);
  GL3_REQUIRE(y_dtype == GL3_F32 || y_dtype == GL3_BF16, "gl3_delta_recurrence: unknown dtype %d", y_dtype);
  // as many waves as the columns need, and as the loads of a chunk of operands need (DR_NLD a thread)
  // the read-outs' norm: by the block that made them where a sequence brings few tokens (a decode step), else by a
  // launch of its own with a wave to every token and head (a block's few waves would walk a prompt's tokens one by one)
  const int norm_here = T <= 4 * B;
  // a column's rows over 8 lanes for prompts (long chains of tokens: half the work per token and wave) where that
  // makes at most eight waves, over 4 else (values of 128: sixteen waves of 8 columns were 5% slower than eight of 16)
  const int rg = (!norm_here && D >= 32 && Dv <= 64) ? 8 : 4;
  const int cols = 64 / rg;
  // (fewer tokens a chunk where that keeps the block at the waves its columns need, or at four)
  // (A head's columns could be dealt out to several blocks, grid z; with blocks of four waves of 8 columns a prompt of
  // 2,048 tokens was slower than with one block of eight, 12.8 against 12.1 ms for sixteen layers: every block stages
  // all of a token's operands, in shorter chunks. One block a head.)
  const int all_col_waves = (Dv + cols - 1) / cols;
  const int col_waves = all_col_waves;
  const int split = 1;
  int chunk = DR_CHUNK, waves = col_waves;
  for (;; chunk /= 2) {
    waves = col_waves;
    while (waves * 64 * DR_NLD < chunk * (2 * D + Dv + 2)) ++waves;
    if (waves <= (col_waves > 4 ? col_waves : 4) || chunk == 1) break;
  }
  GL3_REQUIRE(waves <= 16, "gl3_delta_recurrence: keys of %d with values of %d need more than a block's threads", D, Dv);
  dim3 grid(H, B, split), block(waves * 64);
  const int rows = (D + rg - 1) / rg;
  const int rpl = rows <= 4 ? 4 : rows <= 8 ? 8 : rows <= 16 ? 16 : rows <= 24 ? 24 : rows <= 32 ? 32 : rows <= 48 ? 48 : 64;
  const size_t lds = 2 * (size_t)chunk * (2 * rg * rpl + ((Dv + 2 + 3) & ~3)) * sizeof(float);
  GL3_REQUIRE(lds <= 64 * 1024, "gl3_delta_recurrence: a chunk's operands of %zu bytes exceed shared memory", lds);
#define GO4(R, TO, MAXT, RGV)                                                                                                  \
  delta_recurrence_kernel<R, TO, MAXT, RGV><<<grid, block, lds, stream>>>(act, gates, state, cu_seqlens, slot_ids, o, proj, ldp, \
                                                                          off_gate, norm_w, (TO*)y, eps, s, chunk, norm_here, col_waves)
#define GO3(R, TO, MAXT)                                                       \
  do {                                                                         \
    if constexpr (R <= 32) {                                                   \
      if (rg == 8) { GO4(R, TO, MAXT, 8); break; }                             \
    }                                                                          \
    GO4(R, TO, MAXT, 4);                                                       \
  } while (0)
#define GO2(R, TO)                                                             \
  do {                                                                         \
    if (waves <= 4) GO3(R, TO, 256);                                           \
    else if (waves <= 8) GO3(R, TO, 512);                                      \
    else GO3(R, TO, 1024);                                                     \
  } while (0)
#define GO(R)                                                                  \
  do {                                                                         \
    if (y_dtype == GL3_F32) GO2(R, float);                                     \
    else GO2(R, bf16_t);                                                       \
  } while (0)
  switch (rpl) {
    case 4: GO(4); break;
    case 8: GO(8); break;
    case 16: GO(16); break;
    case 24: GO(24); break;
    case 32: GO(32); break;
    case 48: GO(48); break;
    default: GO(64); break;
  }
#undef GO
#undef GO2
#undef GO3
#undef GO4
  GL3_LAUNCH_CHECK();
  if (!norm_here) {
    GL3_REQUIRE(T <= 2147483647 / 64, "gl3_delta_recurrence: %d tokens exceed the grid", T);
    if (y_dtype == GL3_F32)
      delta_gated_norm_kernel<float><<<dim3(T, H), dim3(64), 0, stream>>>(o, proj, ldp, off_gate, norm_w, (float*)y, H, Dv, eps);
    else
      delta_gated_norm_kernel<bf16_t><<<dim3(T, H), dim3(64), 0, stream>>>(o, proj, ldp, off_gate, norm_w, (bf16_t*)y, H, Dv, eps);
  }
  GL3_LAUNCH_CHECK();
  return 0;
}
