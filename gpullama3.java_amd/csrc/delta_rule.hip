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
// Three launches: delta_prep (convolution, silu, unit length, decay and strength; then the convolution's new
// state), delta_recurrence (the rule itself), delta_gated_norm (each head's read-out divided by its root mean
// square, times a weight shared by the heads, times silu of a gate).
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
__global__ __launch_bounds__(64) void delta_prep_kernel(
    const float* __restrict__ proj, const float* __restrict__ conv_w, const float* __restrict__ A_log,
    const float* __restrict__ dt_bias, const float* __restrict__ state, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_of_token, const int* __restrict__ slot_ids, float* __restrict__ act,
    float* __restrict__ gates, DeltaShape s, float unit_eps, float q_scale) {
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
  const float* held = state + (long)slot_ids[b] * s.state_stride + s.conv_off;
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

// grid (ceil(Dv / 16), H, B), one wave: lane (r, c) holds rows r, r + 4, ... of column c of the tile. RPL: rows a lane.
template <int RPL>
__global__ __launch_bounds__(64) void delta_recurrence_kernel(const float* __restrict__ act, const float* __restrict__ gates,
                                                              float* __restrict__ state, const int* __restrict__ cu_seqlens,
                                                              const int* __restrict__ slot_ids, float* __restrict__ out,
                                                              DeltaShape s) {
  const int ct = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int lane = threadIdx.x, r = lane >> 4, c = lane & 15;
  const int j = ct * 16 + c;
  const bool valid = j < s.Dv;
  const int D = s.D, H = s.H;
  const int C = 2 * s.G * D + H * s.Dv;
  const int kvh = h / (H / s.G);
  const int first = cu_seqlens[b], last = cu_seqlens[b + 1];
  if (last <= first) return;
  const int CT = (s.Dv + 15) / 16;
  float* tile = state + (long)slot_ids[b] * s.state_stride + ((long)(h * CT + ct) * D) * 16;
  float S[RPL];
#pragma unroll
  for (int ii = 0; ii < RPL; ++ii) {
    const int i = r + 4 * ii;
    S[ii] = i < D ? tile[(long)i * 16 + c] : 0.f;
  }
  const long q_at = (long)kvh * D, k_at = (long)s.G * D + (long)kvh * D, v_at = 2L * s.G * D + (long)h * s.Dv + (valid ? j : 0);
  float kr[RPL], qr[RPL], v, g, beta;
  auto fetch = [&](int t) {
    const float* a = act + (long)t * C;
#pragma unroll
    for (int ii = 0; ii < RPL; ++ii) {
      const int i = r + 4 * ii;
      kr[ii] = i < D ? a[k_at + i] : 0.f;
      qr[ii] = i < D ? a[q_at + i] : 0.f;
    }
    v = a[v_at];
    g = gates[(long)t * 2 * H + h];
    beta = gates[(long)t * 2 * H + H + h];
  };
  fetch(first);
  for (int t = first; t < last; ++t) {
    float kc[RPL], qc[RPL];
#pragma unroll
    for (int ii = 0; ii < RPL; ++ii) { kc[ii] = kr[ii]; qc[ii] = qr[ii]; }
    const float vc = v, gc = g, bc = beta;
    if (t + 1 < last) fetch(t + 1);          // the next token's operands travel while this one is worked on
    float part = 0.f;
#pragma unroll
    for (int ii = 0; ii < RPL; ++ii) {
      S[ii] *= gc;
      part = fmaf(S[ii], kc[ii], part);
    }
    part += __shfl_xor(part, 16, 64);
    part += __shfl_xor(part, 32, 64);
    const float uu = bc * (vc - part);
    float o = 0.f;
#pragma unroll
    for (int ii = 0; ii < RPL; ++ii) {
      S[ii] = fmaf(kc[ii], uu, S[ii]);
      o = fmaf(S[ii], qc[ii], o);
    }
    o += __shfl_xor(o, 16, 64);
    o += __shfl_xor(o, 32, 64);
    if (r == 0 && valid) out[(long)t * H * s.Dv + (long)h * s.Dv + j] = o;
  }
#pragma unroll
  for (int ii = 0; ii < RPL; ++ii) {
    const int i = r + 4 * ii;
    if (i < D) tile[(long)i * 16 + c] = S[ii];
  }
}

// grid (T, H), one wave: out[t, h, :] = o / sqrt(mean(o^2) + eps) * w * silu(gate[t, h, :])
template <typename TW, typename TO>
__global__ __launch_bounds__(64) void delta_gated_norm_kernel(const float* __restrict__ o, const float* __restrict__ proj,
                                                              int ldp, int off_gate, const TW* __restrict__ w,
                                                              TO* __restrict__ out, int H, int Dv, float eps) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + ((long)t * H + h) * Dv;
  const float* grow = proj + (long)t * ldp + off_gate + (long)h * Dv;
  float ss = 0.f;
  for (int e = lane; e < Dv; e += 64) ss = fmaf(orow[e], orow[e], ss);
  ss = wave_sum(ss);
  const float f = 1.0f / sqrtf(ss / (float)Dv + eps);
  TO* dst = out + ((long)t * H + h) * Dv;
  for (int e = lane; e < Dv; e += 64) {
    const float z = grow[e];
    dst[e] = from_f32<TO>(orow[e] * f * to_f32<TW>(w[e]) * (z * dr_sigmoid(z)));
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
// state [slots][state_stride] float. act [T][C] and gates [T][2 H] float are written; then the held inputs move on.
extern "C" int gl3_delta_prep(const float* proj, const float* conv_w, const float* A_log, const float* dt_bias,
                              float* state, const int* cu_seqlens, const int* seq_of_token, const int* slot_ids,
                              float* act, float* gates, int T, int B, int H, int G, int D, int Dv, int taps, int ldp,
                              int off_q, int off_k, int off_v, int off_b, int off_a, long state_stride, float unit_eps,
                              float q_scale, hipStream_t stream) {
  if (T == 0 || B == 0) return 0;
  GL3_REQUIRE(proj && conv_w && A_log && dt_bias && state && cu_seqlens && seq_of_token && slot_ids && act && gates &&
                  T > 0 && B > 0, "gl3_delta_prep: bad arguments");
  DeltaShape s;
  if (delta_shape(s, H, G, D, Dv, taps, ldp, off_q, off_k, off_v, off_b, off_a, state_stride)) return -1;
  GL3_REQUIRE(2 * G + H + 1 <= 65535 && B <= 65535, "gl3_delta_prep: too many heads or sequences for the grid");
  delta_prep_kernel<<<dim3(T, 2 * G + H + 1), dim3(64), 0, stream>>>(proj, conv_w, A_log, dt_bias, state, cu_seqlens,
                                                                     seq_of_token, slot_ids, act, gates, s, unit_eps, q_scale);
  GL3_LAUNCH_CHECK();
  if (taps > 1) {
    const int C = 2 * G * D + H * Dv;
    delta_conv_state_kernel<<<dim3(B, (C + 255) / 256), dim3(256), 0, stream>>>(proj, state, cu_seqlens, slot_ids, s);
    GL3_LAUNCH_CHECK();
  }
  return 0;
}

// act [T][C], gates [T][2 H] as gl3_delta_prep left them; out [T][H Dv] float.
extern "C" int gl3_delta_recurrence(const float* act, const float* gates, float* state, const int* cu_seqlens,
                                    const int* slot_ids, float* out, int B, int H, int G, int D, int Dv, int taps,
                                    long state_stride, hipStream_t stream) {
  if (B == 0) return 0;
  GL3_REQUIRE(act && gates && state && cu_seqlens && slot_ids && out && B > 0, "gl3_delta_recurrence: bad arguments");
  DeltaShape s;
  if (delta_shape(s, H, G, D, Dv, taps, 1 << 30, 0, 0, 0, 0, 0, state_stride)) return -1;
  GL3_REQUIRE(H <= 65535 && B <= 65535, "gl3_delta_recurrence: too many heads or sequences for the grid");
  dim3 grid((Dv + 15) / 16, H, B), block(64);
  const int rows = (D + 3) / 4;
#define GO(R) delta_recurrence_kernel<R><<<grid, block, 0, stream>>>(act, gates, state, cu_seqlens, slot_ids, out, s)
  if (rows <= 4) GO(4);
  else if (rows <= 8) GO(8);
  else if (rows <= 16) GO(16);
  else if (rows <= 24) GO(24);
  else if (rows <= 32) GO(32);
  else if (rows <= 48) GO(48);
  else GO(64);
#undef GO
  GL3_LAUNCH_CHECK();
  return 0;
}

// o [T][H Dv] float; proj [T][ldp] float with the gate's H Dv columns from off_gate on; w [Dv]; out [T][H Dv].
extern "C" int gl3_delta_gated_norm(const float* o, const float* proj, int ldp, int off_gate, const void* w, int w_dtype,
                                    void* out, int out_dtype, int T, int H, int Dv, float eps, hipStream_t stream) {
  if (T == 0) return 0;
  GL3_REQUIRE(o && proj && w && out && T > 0 && H > 0 && H <= 65535 && Dv > 0 && off_gate >= 0 && off_gate + H * Dv <= ldp,
              "gl3_delta_gated_norm: bad arguments");
  dim3 grid(T, H), block(64);
#define GO(TW, TO) delta_gated_norm_kernel<TW, TO><<<grid, block, 0, stream>>>(o, proj, ldp, off_gate, (const TW*)w, (TO*)out, H, Dv, eps)
  if (w_dtype == GL3_F32 && out_dtype == GL3_F32) GO(float, float);
  else if (w_dtype == GL3_F32 && out_dtype == GL3_BF16) GO(float, bf16_t);
  else if (w_dtype == GL3_BF16 && out_dtype == GL3_F32) GO(bf16_t, float);
  else if (w_dtype == GL3_BF16 && out_dtype == GL3_BF16) GO(bf16_t, bf16_t);
  else GL3_REQUIRE(false, "gl3_delta_gated_norm: unknown dtypes %d %d", w_dtype, out_dtype);
#undef GO
  GL3_LAUNCH_CHECK();
  return 0;
}
