// Kernels of mixers that keep a state per sequence instead of (or beside) a cache of keys and values, and of what
// stands around them: a hashed second embedding row, the mixture of the residual rows with the embedding's output,
// rotations of whole heads in place, a gate per head, the average of two normalised rows.
// Everything here computes in 32-bit; only what is handed to a matrix product is stored in the activations' type.
#include "common.h"

// ----------------------------------------------------------------- the row of a table of token pairs
// rows[t] = (previous token * mul_prev + token * mul_cur) mod buckets, or `buckets` (the table's last row) for a
// sequence's first token. The previous token of a step's first token is what the sequence's slot holds (held[0] of
// its row of `state`); the thread of that first token also leaves the step's last token there, after it has read, so
// no other thread touches the slot's row.
__global__ void pair_rows_kernel(const int* __restrict__ token_ids, const int* __restrict__ positions,
                                 const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
                                 const int* __restrict__ slot_ids, int* __restrict__ state, long state_stride,
                                 long mul_prev, long mul_cur, long buckets, int* __restrict__ rows, int n_tokens) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n_tokens) return;
  const int seq = seq_of_token[t];
  const int first = cu_seqlens[seq], last = cu_seqlens[seq + 1] - 1;
  int* held = state + (long)slot_ids[seq] * state_stride;
  const long prev = t > first ? token_ids[t - 1] : held[0];
  rows[t] = positions[t] == 0 ? (int)buckets : (int)((prev * mul_prev + (long)token_ids[t] * mul_cur) % buckets);
  if (t == first) held[0] = token_ids[last];
}

extern "C" int gl3_pair_rows(const int* token_ids, const int* positions, const int* seq_of_token, const int* cu_seqlens,
                             const int* slot_ids, int* state, long state_stride, long mul_prev, long mul_cur, long buckets,
                             int* rows, int n_tokens, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(token_ids && positions && seq_of_token && cu_seqlens && slot_ids && state && rows && n_tokens > 0,
              "gl3_pair_rows: bad arguments");
  GL3_REQUIRE(buckets > 0 && buckets < (1L << 31) && mul_prev >= 0 && mul_prev < (1L << 31) && mul_cur >= 0 &&
                  mul_cur < (1L << 31) && state_stride > 0,
              "gl3_pair_rows: %ld buckets, multipliers %ld and %ld", buckets, mul_prev, mul_cur);
  pair_rows_kernel<<<dim3((n_tokens + 255) / 256), dim3(256), 0, stream>>>(
      token_ids, positions, seq_of_token, cu_seqlens, slot_ids, state, state_stride, mul_prev, mul_cur, buckets, rows,
      n_tokens);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- [x; x0] as a product's input
template <typename T>
__global__ void concat_rows_kernel(const float* __restrict__ a, const float* __restrict__ b, T* __restrict__ out, long n, int d) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long t = i / d;
  const int c = (int)(i - t * d);
  out[t * 2 * d + c] = from_f32<T>(a[i]);
  out[t * 2 * d + d + c] = from_f32<T>(b[i]);
}

extern "C" int gl3_concat_rows(const float* a, const float* b, void* out, int out_dtype, int n_tokens, int d,
                               hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(a && b && out && n_tokens > 0 && d > 0, "gl3_concat_rows: bad arguments");
  const long n = (long)n_tokens * d;
  const long blocks = (n + 255) / 256;
  GL3_REQUIRE(blocks < (1L << 31), "gl3_concat_rows: %ld elements is too many", n);
  if (out_dtype == GL3_F32)
    concat_rows_kernel<float><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a, b, (float*)out, n, d);
  else if (out_dtype == GL3_BF16)
    concat_rows_kernel<bf16_t><<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(a, b, (bf16_t*)out, n, d);
  else GL3_REQUIRE(false, "gl3_concat_rows: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- heads turned in place
// Up to three runs of heads inside rows [T][ld] (queries, keys, values of one projection, or one run: an attention's
// output) are rotated by the token's position: the first rot_dim elements of every head as pairs (j, j + rot_dim/2)
// (or (2j, 2j+1)), by the angle whose cos and sin stand in the run's table [position][rot_dim/2]; `back` turns by
// minus the angle. With `gate` (rows [T][gate_ld] of the same type, head h's value at column gate_col + h; one run
// only) every element of head h, rotated or not, is multiplied by sigmoid(gate) afterwards.
struct RotRun {
  int col, heads, head_dim, rot_dim;
  const float* cos_tab;
  const float* sin_tab;
};

template <typename T>
__global__ __launch_bounds__(64) void rotate_heads_kernel(T* __restrict__ rows, long ld, const int* __restrict__ positions,
                                                           RotRun a, RotRun b, RotRun c, int adjacent, int back,
                                                           const T* __restrict__ gate, long gate_ld, int gate_col) {
  const int t = blockIdx.x;
  int head = blockIdx.y;
  RotRun r = a;
  if (head >= a.heads) {
    head -= a.heads;
    r = b;
    if (head >= b.heads) {
      head -= b.heads;
      r = c;
    }
  }
  const int pos = positions[t];
  T* p = rows + (long)t * ld + r.col + (long)head * r.head_dim;
  const int half = r.rot_dim / 2;
  const float g = gate ? 1.0f / (1.0f + expf(-to_f32<T>(gate[(long)t * gate_ld + gate_col + head]))) : 1.0f;
  if (r.cos_tab) {
    for (int j = threadIdx.x; j < half; j += 64) {
      const int i0 = adjacent ? 2 * j : j, i1 = adjacent ? 2 * j + 1 : j + half;
      const float cs = r.cos_tab[(long)pos * half + j];
      const float sn = back ? -r.sin_tab[(long)pos * half + j] : r.sin_tab[(long)pos * half + j];
      const float v0 = to_f32<T>(p[i0]), v1 = to_f32<T>(p[i1]);
      p[i0] = from_f32<T>((v0 * cs - v1 * sn) * g);
      p[i1] = from_f32<T>((v1 * cs + v0 * sn) * g);
    }
  }
  if (gate)
    for (int i = (r.cos_tab ? r.rot_dim : 0) + threadIdx.x; i < r.head_dim; i += 64) p[i] = from_f32<T>(to_f32<T>(p[i]) * g);
}

extern "C" int gl3_rotate_heads(void* rows, int dtype, long ld, const int* positions, int n_tokens, const int* cols,
                                const int* heads, const int* head_dims, const int* rot_dims, const float* const* cos_tabs,
                                const float* const* sin_tabs, int n_runs, int adjacent, int back, const void* gate,
                                long gate_ld, int gate_col, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(rows && positions && n_tokens > 0 && n_runs >= 1 && n_runs <= 3, "gl3_rotate_heads: bad arguments");
  GL3_REQUIRE(!gate || n_runs == 1, "gl3_rotate_heads: a gate goes with one run of heads");
  RotRun r[3] = {};
  long total = 0;
  for (int i = 0; i < n_runs; ++i) {
    r[i] = RotRun{cols[i], heads[i], head_dims[i], rot_dims[i], cos_tabs[i], sin_tabs[i]};
    GL3_REQUIRE(heads[i] > 0 && head_dims[i] > 0 && rot_dims[i] >= 0 && rot_dims[i] % 2 == 0 && rot_dims[i] <= head_dims[i] &&
                    cols[i] >= 0 && cols[i] + (long)heads[i] * head_dims[i] <= ld && (cos_tabs[i] == nullptr) == (sin_tabs[i] == nullptr),
                "gl3_rotate_heads: run %d: %d heads of %d (%d rotated) from column %d of rows of %ld", i, heads[i],
                head_dims[i], rot_dims[i], cols[i], ld);
    total += heads[i];
  }
  GL3_REQUIRE(total <= 65535, "gl3_rotate_heads: %ld heads exceed the grid", total);
  dim3 grid(n_tokens, (unsigned)total), block(64);
  if (dtype == GL3_F32)
    rotate_heads_kernel<float><<<grid, block, 0, stream>>>((float*)rows, ld, positions, r[0], r[1], r[2], adjacent, back,
                                                           (const float*)gate, gate_ld, gate_col);
  else if (dtype == GL3_BF16)
    rotate_heads_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)rows, ld, positions, r[0], r[1], r[2], adjacent, back,
                                                            (const bf16_t*)gate, gate_ld, gate_col);
  else GL3_REQUIRE(false, "gl3_rotate_heads: unknown dtype %d", dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- x += f * (a / rms(a) * wa + b / rms(b) * wb)
// One block a token. `b` may be null (one side only). Sums in an order that depends on d alone.
__global__ __launch_bounds__(256) void sides_norm_add_kernel(float* __restrict__ x, const float* __restrict__ a,
                                                              const float* __restrict__ b, const float* __restrict__ wa,
                                                              const float* __restrict__ wb, float eps, float f, int d) {
  __shared__ float scratch[16];
  const long t = blockIdx.x;
  const float* pa = a + t * d;
  const float* pb = b ? b + t * d : nullptr;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < d; i += 256) {
    const float va = pa[i];
    sa += va * va;
    if (pb) {
      const float vb = pb[i];
      sb += vb * vb;
    }
  }
  sa = block_sum(sa, scratch);
  sb = block_sum(sb, scratch);
  const float ia = 1.0f / sqrtf(sa / (float)d + eps), ib = 1.0f / sqrtf(sb / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += 256) {
    float v = pa[i] * ia * wa[i];
    if (pb) v += pb[i] * ib * wb[i];
    x[t * d + i] += f * v;
  }
}

extern "C" int gl3_sides_norm_add(float* x, const float* a, const float* b, const float* wa, const float* wb, float eps,
                                  float f, int n_tokens, int d, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(x && a && wa && (!b || wb) && n_tokens > 0 && d > 0, "gl3_sides_norm_add: bad arguments");
  sides_norm_add_kernel<<<dim3(n_tokens), dim3(256), 0, stream>>>(x, a, b, wa, wb, eps, f, d);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- out = tanh(in) in the activations' type
template <typename T>
__global__ void tanh_rows_kernel(const float* __restrict__ in, T* __restrict__ out, long n) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = from_f32<T>(tanhf(in[i]));
}

extern "C" int gl3_tanh_rows(const float* in, void* out, int out_dtype, long n, hipStream_t stream) {
  if (n == 0) return 0;
  GL3_REQUIRE(in && out && n > 0 && (n + 255) / 256 < (1L << 31), "gl3_tanh_rows: bad arguments");
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (out_dtype == GL3_F32) tanh_rows_kernel<float><<<grid, block, 0, stream>>>(in, (float*)out, n);
  else if (out_dtype == GL3_BF16) tanh_rows_kernel<bf16_t><<<grid, block, 0, stream>>>(in, (bf16_t*)out, n);
  else GL3_REQUIRE(false, "gl3_tanh_rows: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- minGRU
// proj [T][ld] float: columns 0 .. W the update gate's sums (biased), W .. 2W the candidate's, 2W .. 3W the output
// gate's. Per sequence and channel, token by token from the state in the sequence's slot:
//   z = sigmoid(pz); c = pu >= 0 ? pu + 1/2 : sigmoid(pu); S = (1 - z) S + z c; out = S * silu(pg).
// grid (channels / 256, sequences). A step's tokens of one sequence are walked in order, so every cut of a
// sequence into steps gives the same numbers.
template <typename TO>
__global__ __launch_bounds__(256) void mingru_scan_kernel(const float* __restrict__ proj, long ld, int W,
                                                           float* __restrict__ state, long state_stride,
                                                           const int* __restrict__ cu_seqlens,
                                                           const int* __restrict__ slot_ids, TO* __restrict__ out) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= W) return;
  const int seq = blockIdx.y;
  float* held = state + (long)slot_ids[seq] * state_stride + c;
  float S = *held;
  const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const float* p = proj + (long)t * ld + c;
    const float pz = p[0], pu = p[W], pg = p[2 * W];
    const float z = 1.0f / (1.0f + expf(-pz));
    const float cand = pu >= 0.f ? pu + 0.5f : 1.0f / (1.0f + expf(-pu));
    S = (1.0f - z) * S + z * cand;
    out[(long)t * W + c] = from_f32<TO>(S * (pg / (1.0f + expf(-pg))));
  }
  *held = S;
}

extern "C" int gl3_mingru_scan(const float* proj, long ld, int W, float* state, long state_stride, const int* cu_seqlens,
                               const int* slot_ids, void* out, int out_dtype, int n_seqs, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  GL3_REQUIRE(proj && state && cu_seqlens && slot_ids && out && W > 0 && ld >= 3L * W && state_stride >= W &&
                  n_seqs > 0 && n_seqs <= 65535, "gl3_mingru_scan: bad arguments (W=%d ld=%ld B=%d)", W, ld, n_seqs);
  dim3 grid((W + 255) / 256, n_seqs), block(256);
  if (out_dtype == GL3_F32)
    mingru_scan_kernel<float><<<grid, block, 0, stream>>>(proj, ld, W, state, state_stride, cu_seqlens, slot_ids, (float*)out);
  else if (out_dtype == GL3_BF16)
    mingru_scan_kernel<bf16_t><<<grid, block, 0, stream>>>(proj, ld, W, state, state_stride, cu_seqlens, slot_ids, (bf16_t*)out);
  else GL3_REQUIRE(false, "gl3_mingru_scan: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- blends with the previous token's row
// out[s][t] = h[t] + (h'[t] - h[t]) * mu[s] for s < n_mix, h' the row of the token before t in its sequence: row
// t - 1 of the step, or for a step's first token what the sequence's slot holds (zeros at a sequence's start).
// `inline_update` (every sequence brings one token): the thread that read element i of the held row writes the
// token's own there; otherwise gl3_keep_last_rows runs after this kernel.
template <typename T>
__global__ __launch_bounds__(256) void shift_mix_kernel(const T* __restrict__ h, int d, const float* __restrict__ mu,
                                                         int n_mix, float* __restrict__ state, long state_stride,
                                                         const int* __restrict__ cu_seqlens,
                                                         const int* __restrict__ seq_of_token,
                                                         const int* __restrict__ slot_ids, T* __restrict__ out,
                                                         long n_tokens, int inline_update) {
  const long t = blockIdx.x;
  const int seq = seq_of_token[t];
  const bool from_step = t > cu_seqlens[seq];
  float* held = state + (long)slot_ids[seq] * state_stride;
  for (int i = threadIdx.x; i < d; i += 256) {
    const float cur = to_f32<T>(h[t * d + i]);
    const float prev = from_step ? to_f32<T>(h[(t - 1) * d + i]) : held[i];
    const float diff = prev - cur;
    for (int s = 0; s < n_mix; ++s) out[((long)s * n_tokens + t) * d + i] = from_f32<T>(cur + diff * mu[(long)s * d + i]);
    if (inline_update) held[i] = cur;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void keep_last_rows_kernel(const T* __restrict__ h, int d, float* __restrict__ state,
                                                              long state_stride, const int* __restrict__ cu_seqlens,
                                                              const int* __restrict__ slot_ids) {
  const int seq = blockIdx.x;
  const long last = cu_seqlens[seq + 1] - 1;
  if (last < cu_seqlens[seq]) return;
  float* held = state + (long)slot_ids[seq] * state_stride;
  for (int i = threadIdx.x; i < d; i += 256) held[i] = to_f32<T>(h[last * d + i]);
}

extern "C" int gl3_shift_mix(const void* h, int dtype, int d, const float* mu, int n_mix, float* state, long state_stride,
                             const int* cu_seqlens, const int* seq_of_token, const int* slot_ids, void* out, int n_tokens,
                             int n_seqs, int one_token_each, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(h && mu && state && cu_seqlens && seq_of_token && slot_ids && out && d > 0 && n_mix > 0 && n_tokens > 0 &&
                  n_seqs > 0 && state_stride >= d, "gl3_shift_mix: bad arguments");
  const int inl = one_token_each && n_tokens == n_seqs;
  if (dtype == GL3_F32) {
    shift_mix_kernel<float><<<dim3(n_tokens), dim3(256), 0, stream>>>((const float*)h, d, mu, n_mix, state, state_stride,
                                                                      cu_seqlens, seq_of_token, slot_ids, (float*)out, n_tokens, inl);
    if (!inl) keep_last_rows_kernel<float><<<dim3(n_seqs), dim3(256), 0, stream>>>((const float*)h, d, state, state_stride, cu_seqlens, slot_ids);
  } else if (dtype == GL3_BF16) {
    shift_mix_kernel<bf16_t><<<dim3(n_tokens), dim3(256), 0, stream>>>((const bf16_t*)h, d, mu, n_mix, state, state_stride,
                                                                       cu_seqlens, seq_of_token, slot_ids, (bf16_t*)out, n_tokens, inl);
    if (!inl) keep_last_rows_kernel<bf16_t><<<dim3(n_seqs), dim3(256), 0, stream>>>((const bf16_t*)h, d, state, state_stride, cu_seqlens, slot_ids);
  } else GL3_REQUIRE(false, "gl3_shift_mix: unknown dtype %d", dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- the decayed matrix per head
// Per sequence and head a matrix S [D keys][D values] in 32-bit (state: [H][D][D] floats from `state_off` of the
// slot's row). r, k, v, wl are [T][H*D] float; the decay of key channel i is w = exp(-exp(wl)); bonus [H][D].
//   o_t[j] = sum_i r_t[i] (S[i][j] + bonus[i] k_t[i] v_t[j]);   S[i][j] <- w_t[i] S[i][j] + k_t[i] v_t[j]
// grid (H, sequences). A thread owns RP rows of one column j in registers (D * ceil(D / RP) threads a block); a
// token's r, k, w, v reach the block through shared memory four tokens at a time, the parts of a column's sum are
// added in shared memory in the order of the parts. Tokens are walked in order from the state in the slot.
#define TM_CH 4
#define TM_MAXD 256

template <int RP>
__global__ __launch_bounds__(1024) void timemix_kernel(const float* __restrict__ r, const float* __restrict__ k,
                                                        const float* __restrict__ v, const float* __restrict__ wl,
                                                        const float* __restrict__ bonus, float* __restrict__ state,
                                                        long state_stride, long state_off,
                                                        const int* __restrict__ cu_seqlens,
                                                        const int* __restrict__ slot_ids, float* __restrict__ o, int H,
                                                        int D) {
  __shared__ float sr[TM_CH][TM_MAXD], sk[TM_CH][TM_MAXD], sw[TM_CH][TM_MAXD], sv[TM_CH][TM_MAXD];
  __shared__ float parts[TM_CH][1024];
  __shared__ float su[TM_MAXD];
  const int head = blockIdx.x, seq = blockIdx.y, tid = threadIdx.x, nt = blockDim.x;
  const int j = tid % D, part = tid / D, i0 = part * RP;
  const int P = (D + RP - 1) / RP;
  const long HD = (long)H * D;
  float* held = state + (long)slot_ids[seq] * state_stride + state_off + (long)head * D * D;
  float S[RP];
#pragma unroll
  for (int ii = 0; ii < RP; ++ii) {
    const int i = i0 + ii;
    S[ii] = i < D ? held[(long)i * D + j] : 0.f;
  }
  for (int i = tid; i < D; i += nt) su[i] = bonus[head * D + i];
  const int t0 = cu_seqlens[seq], t1 = cu_seqlens[seq + 1];
  for (int tb = t0; tb < t1; tb += TM_CH) {
    const int n = t1 - tb < TM_CH ? t1 - tb : TM_CH;
    __syncthreads();
    for (int idx = tid; idx < n * D; idx += nt) {
      const int tt = idx / D, i = idx - tt * D;
      const long at = (long)(tb + tt) * HD + head * D + i;
      sr[tt][i] = r[at];
      sk[tt][i] = k[at];
      sv[tt][i] = v[at];
      sw[tt][i] = expf(-expf(wl[at]));
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float vj = sv[tt][j];
      float acc = 0.f;
#pragma unroll
      for (int ii = 0; ii < RP; ++ii) {
        const int i = i0 + ii;
        if (i < D) {
          const float kv = sk[tt][i] * vj;
          acc = fmaf(sr[tt][i], S[ii] + su[i] * kv, acc);
          S[ii] = sw[tt][i] * S[ii] + kv;
        }
      }
      parts[tt][tid] = acc;
    }
    __syncthreads();
    for (int idx = tid; idx < n * D; idx += nt) {
      const int tt = idx / D, jj = idx - tt * D;
      float sum = 0.f;
      for (int p = 0; p < P; ++p) sum += parts[tt][p * D + jj];
      o[(long)(tb + tt) * HD + head * D + jj] = sum;
    }
  }
#pragma unroll
  for (int ii = 0; ii < RP; ++ii) {
    const int i = i0 + ii;
    if (i < D) held[(long)i * D + j] = S[ii];
  }
}

extern "C" int gl3_timemix(const float* r, const float* k, const float* v, const float* wl, const float* bonus,
                           float* state, long state_stride, long state_off, const int* cu_seqlens, const int* slot_ids,
                           float* o, int n_seqs, int H, int D, hipStream_t stream) {
  if (n_seqs == 0) return 0;
  GL3_REQUIRE(r && k && v && wl && bonus && state && cu_seqlens && slot_ids && o && n_seqs > 0 && n_seqs <= 65535 && H > 0,
              "gl3_timemix: bad arguments");
  GL3_REQUIRE(D >= 1 && D <= TM_MAXD, "gl3_timemix: heads of %d elements: the kernel holds up to %d", D, TM_MAXD);
  GL3_REQUIRE(state_off >= 0 && state_off + (long)H * D * D <= state_stride, "gl3_timemix: the state's row of %ld floats", state_stride);
  dim3 grid(H, n_seqs);
  if (D <= 128) {
    const int P = (D + 15) / 16;
    timemix_kernel<16><<<grid, dim3(D * P), 0, stream>>>(r, k, v, wl, bonus, state, state_stride, state_off, cu_seqlens,
                                                        slot_ids, o, H, D);
  } else {
    const int P = (D + 63) / 64;
    timemix_kernel<64><<<grid, dim3(D * P), 0, stream>>>(r, k, v, wl, bonus, state, state_stride, state_off, cu_seqlens,
                                                        slot_ids, o, H, D);
  }
  GL3_LAUNCH_CHECK();
  return 0;
}

// ----------------------------------------------------------------- a norm per head, a weight per channel, a gate
// out[t, h, i] = o[t, h, i] / sqrt(mean_i(o[t, h]^2) + eps) * w[h * D + i] * silu(gate[t, h * D + i]); one wave a
// (token, head).
template <typename TO>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             const float* __restrict__ gate, float eps,
                                                             TO* __restrict__ out, int H, int D) {
  const long base = ((long)blockIdx.x * H + blockIdx.y) * D;
  const int wbase = blockIdx.y * D;
  float ss = 0.f;
  for (int i = threadIdx.x; i < D; i += 64) {
    const float x = o[base + i];
    ss += x * x;
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)D + eps);
  for (int i = threadIdx.x; i < D; i += 64) {
    const float g = gate[base + i];
    out[base + i] = from_f32<TO>(o[base + i] * inv * w[wbase + i] * (g / (1.0f + expf(-g))));
  }
}

extern "C" int gl3_head_norm_gate(const float* o, const float* w, const float* gate, float eps, void* out, int out_dtype,
                                  int n_tokens, int H, int D, hipStream_t stream) {
  if (n_tokens == 0) return 0;
  GL3_REQUIRE(o && w && gate && out && n_tokens > 0 && H > 0 && H <= 65535 && D > 0, "gl3_head_norm_gate: bad arguments");
  dim3 grid(n_tokens, H), block(64);
  if (out_dtype == GL3_F32) head_norm_gate_kernel<float><<<grid, block, 0, stream>>>(o, w, gate, eps, (float*)out, H, D);
  else if (out_dtype == GL3_BF16) head_norm_gate_kernel<bf16_t><<<grid, block, 0, stream>>>(o, w, gate, eps, (bf16_t*)out, H, D);
  else GL3_REQUIRE(false, "gl3_head_norm_gate: unknown dtype %d", out_dtype);
  GL3_LAUNCH_CHECK();
  return 0;
}
