// Recurrences with a diagonal decay: linear attention whose heads forget at a fixed rate each, and the selective
// scan (a state per channel whose step size depends on the token), with the short causal convolution in front of it.
//
// Everything that enters a recurrence is 32-bit: the state, step sizes, decays and their exponentials.  A request's
// state is one row of a `[slots + 1, floats]` tensor; an entry that starts at position 0 treats its row as zeros, so
// a slot that is used again needs no clearing.  The tokens of a step lie flat, entry after entry; `entry_start[e]`
// is the first token of entry e, `entry_first[e]` its position in the request, `slots[e]` the state row.
//
// Both recurrences give the sixteen lanes of a quarter of a wave one output channel: each lane keeps R of the
// channel's state numbers in registers, a sum over the state is R terms in a lane in ascending order and then four
// DPP exchanges inside the sixteen lanes.  That order depends on the sizes alone, so a token's result does not depend
// on how its prompt was cut or on what else is in the step.  A workgroup is one wave: four channels of one entry,
// whose tokens it walks in order, a few tokens' operands on their way while the few before them are worked on; no
// load sits behind a branch (a token past the entry's end reads the last one again).  What does not depend on the
// state (activations of the inputs, the step sizes' softplus) is taken inside for steps of single tokens and once,
// by a kernel ahead, for a prompt's portion, where every wave would pay for it token behind token.
#include "common.h"

__device__ __forceinline__ float scan_silu(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float scan_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float scan_softplus(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

template <int CTRL>
__device__ __forceinline__ float scan_dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false);
  return v + __int_as_float(moved);
}

// The sum over the 16 lanes of a row, in every lane, without LDS: neighbours, pairs of neighbours, the other quad of
// the eight, the other eight.
__device__ __forceinline__ float row16_sum(float v) {
  v = scan_dpp_add<0xB1>(v);     // quad_perm [1, 0, 3, 2]
  v = scan_dpp_add<0x4E>(v);     // quad_perm [2, 3, 0, 1]
  v = scan_dpp_add<0x141>(v);    // row_half_mirror
  v = scan_dpp_add<0x140>(v);    // row_mirror
  return v;
}

constexpr int SCAN_THREADS = 64;      // a workgroup is one wave: four channels of sixteen lanes
constexpr int SCAN_CHANNELS = 4;

static inline int lanes_share(int n) { return n <= 16 ? 1 : n <= 32 ? 2 : n <= 64 ? 4 : n <= 128 ? 8 : 16; }

// ---------------------------------------------------------------------------------------------
// Linear attention with a fixed decay per head:  S <- decay_h S + k v^T,  o = S^T q   (S is dim x vdim).
//   q, k  [T, ldqk] 32-bit, head h at columns h * dim;  v [T, ldv], head h at columns h * vdim
//   act   1: q, k and v pass through silu as they are read
//   state per head `vdim * 16 R` floats: value channel c holds its key channels, padded to 16 R, one after another
// Grid (entries, heads, ceil(vdim / 4)).  VEC: dim = 16 R with R a multiple of 4 and 16-byte rows, so a lane's run of
// key channels is read four at a time.
template <int R, bool VEC>
__global__ __launch_bounds__(SCAN_THREADS) void decay_rule_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                         long long ldqk, const float* __restrict__ v, long long ldv,
                                                         int act, const float* __restrict__ decay,
                                                         float* __restrict__ state, long long state_stride,
                                                         const int* __restrict__ entry_start,
                                                         const int* __restrict__ entry_first,
                                                         const int* __restrict__ slots, int heads, int dim, int vdim,
                                                         float* __restrict__ o) {
  const int e = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x & 63;
  const int part = lane & 15;
  const int vch = blockIdx.z * SCAN_CHANNELS + (lane >> 4);
  const bool live = vch < vdim;
  const int vcol = h * vdim + min(vch, vdim - 1);
  const int t0 = entry_start[e], t1 = entry_start[e + 1];
  const bool fresh = entry_first[e] == 0;
  const float rate = decay[h];
  float* row = state + (long long)slots[e] * state_stride + ((long long)h * vdim + min(vch, vdim - 1)) * (16 * R) + part * R;
  float s[R];
  int col[R];
  bool in[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int c = part * R + r;
    in[r] = c < dim;
    col[r] = h * dim + min(c, dim - 1);
    const float old = row[r];
    s[r] = (fresh || !in[r]) ? 0.f : old;
  }
  if (t1 <= t0) return;
  // D tokens' operands are on their way while the D before them are worked on: a token's step is a few dozen
  // instructions, a load's way through the caches several hundred cycles
  constexpr int D = R >= 16 ? 2 : 4;
  float nk[D][R], nq[D][R], nv[D];
  auto fetch = [&](int first) {
#pragma unroll
    for (int j = 0; j < D; ++j) {
      const int t = min(first + j, t1 - 1);
      const float* kr = k + (long long)t * ldqk;
      const float* qr = q + (long long)t * ldqk;
      if constexpr (VEC) {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int r = 0; r < R; r += 4) {
          const f32x4 k4 = *(const f32x4*)(kr + col[r]), q4 = *(const f32x4*)(qr + col[r]);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            nk[j][r + i] = k4[i];
            nq[j][r + i] = q4[i];
          }
        }
      } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          nk[j][r] = kr[col[r]];
          nq[j][r] = qr[col[r]];
        }
      }
      nv[j] = v[(long long)t * ldv + vcol];
    }
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += D) {
    float ck[D][R], cq[D][R], cv[D];
#pragma unroll
    for (int j = 0; j < D; ++j) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        ck[j][r] = nk[j][r];
        cq[j][r] = nq[j][r];
      }
      cv[j] = nv[j];
    }
    fetch(tb + D);
#pragma unroll
    for (int j = 0; j < D; ++j) {
      const int t = tb + j;
      if (t >= t1) break;
      if (act) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          ck[j][r] = scan_silu(ck[j][r]);
          cq[j][r] = scan_silu(cq[j][r]);
        }
        cv[j] = scan_silu(cv[j]);
      }
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float kk = in[r] ? ck[j][r] : 0.f;
        s[r] = fmaf(rate, s[r], kk * cv[j]);
        sum = fmaf(s[r], in[r] ? cq[j][r] : 0.f, sum);
      }
      sum = row16_sum(sum);
      if (part == 0 && live) o[(long long)t * heads * vdim + vcol] = sum;
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r) row[r] = s[r];
  }
}

extern "C" long long vk_decay_rule_head_floats(int dim, int vdim) { return (long long)vdim * 16 * lanes_share(dim); }

extern "C" int vk_decay_rule(const float* q, const float* k, long long ldqk, const float* v, long long ldv, int act,
                             const float* decay, float* state, long long state_stride, const int* entry_start,
                             const int* entry_first, const int* slots, int num_entries, int heads, int dim, int vdim,
                             float* o, void* stream) {
  if (num_entries <= 0) return 0;
  if (heads < 1 || dim < 1 || vdim < 1 || heads > 65535) return VK_BAD_ARGUMENT;
  if (dim > 256) return VK_UNSUPPORTED_SIZE;
  if (state_stride < heads * vk_decay_rule_head_floats(dim, vdim)) return VK_BAD_ARGUMENT;
  dim3 grid(num_entries, heads, (vdim + SCAN_CHANNELS - 1) / SCAN_CHANNELS);
  if (grid.z > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  const int share = lanes_share(dim);
  const bool vec = share >= 4 && dim == 16 * share && ldqk % 4 == 0 && (((uintptr_t)q | (uintptr_t)k) & 15) == 0;
#define VK_DR(RR, VV)                                                                                                 \
  decay_rule_kernel<RR, VV><<<grid, SCAN_THREADS, 0, s>>>(q, k, ldqk, v, ldv, act, decay, state, state_stride,        \
                                                          entry_start, entry_first, slots, heads, dim, vdim, o)
  switch (share) {
    case 1: VK_DR(1, false); break;
    case 2: VK_DR(2, false); break;
    case 4: if (vec) VK_DR(4, true); else VK_DR(4, false); break;
    case 8: if (vec) VK_DR(8, true); else VK_DR(8, false); break;
    default: if (vec) VK_DR(16, true); else VK_DR(16, false); break;
  }
#undef VK_DR
  VK_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// out[t, c] = x[t, c] / rms(x[t, :]) * weight[c] * gate(g[t, c]) over the whole row; gate_act 0: g as it is,
// 1: silu, 2: sigmoid.  One workgroup per token.
template <typename TO>
__global__ __launch_bounds__(256) void gated_norm_kernel(const float* __restrict__ x, const float* __restrict__ weight,
                                                         const float* __restrict__ gate, long long ldg, int gate_act,
                                                         float eps, int width, TO* __restrict__ out) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* src = x + (long long)t * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) ss += src[c] * src[c];
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int c = threadIdx.x; c < width; c += 256) {
    float g = gate[(long long)t * ldg + c];
    g = gate_act == 1 ? scan_silu(g) : gate_act == 2 ? scan_sigmoid(g) : g;
    out[(long long)t * width + c] = from_float<TO>(src[c] * inv * weight[c] * g);
  }
}

extern "C" int vk_gated_norm(const float* x, const float* weight, const float* gate, long long ldg, int gate_act,
                             float eps, int num_tokens, int width, void* out, int out_dtype, void* stream) {
  if (num_tokens <= 0) return 0;
  if (width < 1 || gate_act < 0 || gate_act > 2) return VK_BAD_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == DT_F32)
    gated_norm_kernel<float><<<num_tokens, 256, 0, s>>>(x, weight, gate, ldg, gate_act, eps, width, (float*)out);
  else if (out_dtype == DT_BF16)
    gated_norm_kernel<bf16_t><<<num_tokens, 256, 0, s>>>(x, weight, gate, ldg, gate_act, eps, width, (bf16_t*)out);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Short causal convolution over time per channel, a bias, then silu:
//   y[t, c] = silu(bias[c] + sum_j conv[c, j] * in[t - (taps - 1 - j), c])
//   in    [T, ldi] 32-bit, channel c at column c; inputs before the entry's first token come from the state row
//         (`(taps - 1) * C` floats from `conv_offset` on, oldest first), or are zero for an entry at position 0
//   conv  [C, taps], the last column is the current token's
// Outputs: y32 [T, C] 32-bit and, if given, the same rounded to TO.  Grid (tokens, ceil(C / 256)).
template <typename TO>
__global__ __launch_bounds__(256) void causal_conv_kernel(const float* __restrict__ in, long long ldi,
                                                          const float* __restrict__ conv,
                                                          const float* __restrict__ bias, int taps, int C,
                                                          const float* __restrict__ state, long long state_stride,
                                                          long long conv_offset, const int* __restrict__ entry_of,
                                                          const int* __restrict__ entry_start,
                                                          const int* __restrict__ entry_first,
                                                          const int* __restrict__ slots, float* __restrict__ y32,
                                                          TO* __restrict__ yrun) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int e = entry_of[t];
  const int offset = t - entry_start[e];
  const bool fresh = entry_first[e] == 0;
  const float* old = state + (long long)slots[e] * state_stride + conv_offset;
  float sum = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;
    const bool in_step = back <= offset, in_state = !in_step && !fresh;
    const float* from = in_step ? in + (long long)(t - back) * ldi + c
                                : in_state ? old + (long long)(taps - 1 - (back - offset)) * C + c : in + (long long)t * ldi + c;
    const float x = *from;
    sum = fmaf(conv[(long long)c * taps + j], (in_step || in_state) ? x : 0.f, sum);
  }
  const float y = scan_silu(sum);
  y32[(long long)t * C + c] = y;
  if (yrun) yrun[(long long)t * C + c] = from_float<TO>(y);
}

// The convolution's inputs of an entry's last taps - 1 tokens become the state; runs after the convolution has read
// the old rows.  Grid (entries, ceil(C / 256)), a thread per channel.
__global__ __launch_bounds__(256) void conv_keep_kernel(const float* __restrict__ in, long long ldi, int taps, int C,
                                                        float* __restrict__ state, long long state_stride,
                                                        long long conv_offset, const int* __restrict__ entry_start,
                                                        const int* __restrict__ entry_first,
                                                        const int* __restrict__ slots) {
  const int e = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int start = entry_start[e], count = entry_start[e + 1] - start;
  if (count <= 0) return;
  const bool fresh = entry_first[e] == 0;
  float* rows = state + (long long)slots[e] * state_stride + conv_offset;
  const int keep = taps - 1;
  for (int j = 0; j < keep; ++j) {           // ascending: row j + count is read before it is written
    const int from = j + count;              // index into [old rows (keep) | the entry's tokens (count)]
    const bool in_step = from >= keep;
    const float* source = in_step ? in + (long long)(start + from - keep) * ldi + c : rows + (long long)from * C + c;
    const float x = *source;
    rows[(long long)j * C + c] = (in_step || !fresh) ? x : 0.f;
  }
}

extern "C" int vk_causal_conv(const float* in, long long ldi, const float* conv, const float* bias, int taps, int C,
                              float* state, long long state_stride, long long conv_offset, const int* entry_of,
                              const int* entry_start, const int* entry_first, const int* slots, int num_tokens,
                              int num_entries, float* y32, void* yrun, int run_dtype, void* stream) {
  if (num_tokens <= 0) return 0;
  if (taps < 1 || C < 1 || num_entries < 1) return VK_BAD_ARGUMENT;
  dim3 grid(num_tokens, (C + 255) / 256);
  if (grid.y > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  if (yrun == nullptr || run_dtype == DT_F32)
    causal_conv_kernel<float><<<grid, 256, 0, s>>>(in, ldi, conv, bias, taps, C, state, state_stride, conv_offset,
                                                   entry_of, entry_start, entry_first, slots, y32, (float*)yrun);
  else if (run_dtype == DT_BF16)
    causal_conv_kernel<bf16_t><<<grid, 256, 0, s>>>(in, ldi, conv, bias, taps, C, state, state_stride, conv_offset,
                                                    entry_of, entry_start, entry_first, slots, y32, (bf16_t*)yrun);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  if (taps > 1) {
    conv_keep_kernel<<<dim3(num_entries, grid.y), 256, 0, s>>>(in, ldi, taps, C, state, state_stride, conv_offset,
                                                               entry_start, entry_first, slots);
    VK_LAUNCH_CHECK();
  }
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Selective scan.  Per channel c and state n:
//   dt = softplus(dtraw[t, c] + dt_bias[c]);  S[c, n] <- exp(dt A[c, n]) S[c, n] + dt x[t, c] B[t, n]
//   y = sum_n S[c, n] C[t, n] + D[c] x[t, c];  out[t, c] = y * silu(z[t, c])
//   A = -exp(a_log) [C, N];  B and C are column ranges of one [T, ldbc] buffer;  z a column range of [T, ldz]
//   state per channel 16 R floats (N padded), channel after channel
//   prepared: dtraw already holds softplus(dt + dt_bias) and z already silu(z) (scan_prepare below; a prompt's tokens
//   would each pay for them behind one another here)
// Grid (entries, ceil(C / 4)).
template <int R, typename TO>
__global__ __launch_bounds__(SCAN_THREADS) void selective_scan_kernel(
    const float* __restrict__ x, const float* __restrict__ dtraw, long long lddt, const float* __restrict__ dt_bias,
    const float* __restrict__ bmat, const float* __restrict__ cmat, long long ldbc, const float* __restrict__ a_log,
    const float* __restrict__ skip, const float* __restrict__ z, long long ldz, float* __restrict__ state,
    long long state_stride, const int* __restrict__ entry_start, const int* __restrict__ entry_first,
    const int* __restrict__ slots, int C, int N, int prepared, TO* __restrict__ out) {
  const int e = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int part = lane & 15;
  const int ch_raw = blockIdx.y * SCAN_CHANNELS + (lane >> 4);
  const bool live = ch_raw < C;
  const int ch = min(ch_raw, C - 1);
  const int t0 = entry_start[e], t1 = entry_start[e + 1];
  const bool fresh = entry_first[e] == 0;
  float* row = state + (long long)slots[e] * state_stride + (long long)ch * (16 * R) + part * R;
  float s[R], a[R];
  int col[R];
  bool in[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int n = part * R + r;
    in[r] = n < N;
    col[r] = min(n, N - 1);
    const float old = row[r];
    s[r] = (fresh || !in[r]) ? 0.f : old;
    a[r] = -expf(a_log[(long long)ch * N + col[r]]);
  }
  if (t1 <= t0) return;
  const float bias = dt_bias[ch], d = skip[ch];
  // D tokens' operands are on their way while the D before them are worked on (see decay_rule_kernel)
  constexpr int D = R >= 8 ? 2 : R >= 4 ? 4 : 8;
  float nb[D][R], nc[D][R], nx[D], ndt[D], nz[D];
  auto fetch = [&](int first) {
#pragma unroll
    for (int j = 0; j < D; ++j) {
      const int t = min(first + j, t1 - 1);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        nb[j][r] = bmat[(long long)t * ldbc + col[r]];
        nc[j][r] = cmat[(long long)t * ldbc + col[r]];
      }
      nx[j] = x[(long long)t * C + ch];
      ndt[j] = dtraw[(long long)t * lddt + ch];
      nz[j] = z[(long long)t * ldz + ch];
    }
  };
  fetch(t0);
  for (int tb = t0; tb < t1; tb += D) {
    float cb[D][R], cc[D][R], cx[D], cdt[D], cz[D];
#pragma unroll
    for (int j = 0; j < D; ++j) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        cb[j][r] = nb[j][r];
        cc[j][r] = nc[j][r];
      }
      cx[j] = nx[j];
      cdt[j] = ndt[j];
      cz[j] = nz[j];
    }
    fetch(tb + D);
#pragma unroll
    for (int j = 0; j < D; ++j) {
      const int t = tb + j;
      if (t >= t1) break;
      const float dt = prepared ? cdt[j] : scan_softplus(cdt[j] + bias);
      const float dtx = dt * cx[j];
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float keep = expf(dt * a[r]);
        s[r] = fmaf(keep, s[r], in[r] ? dtx * cb[j][r] : 0.f);
        sum = fmaf(s[r], in[r] ? cc[j][r] : 0.f, sum);
      }
      sum = row16_sum(sum);
      if (part == 0 && live)
        out[(long long)t * C + ch] = from_float<TO>(fmaf(d, cx[j], sum) * (prepared ? cz[j] : scan_silu(cz[j])));
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r) row[r] = s[r];
  }
}

// dt[t, c] <- softplus(dt[t, c] + dt_bias[c]) in place and gate[t, c] = silu(z[t, c]): what the scan of a prompt's
// portion would otherwise compute token behind token.
__global__ void scan_prepare_kernel(float* __restrict__ dt, long long lddt, const float* __restrict__ dt_bias,
                                    const float* __restrict__ z, long long ldz, float* __restrict__ gate, int C,
                                    long long total) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long t = idx / C;
  const int c = (int)(idx % C);
  dt[t * lddt + c] = scan_softplus(dt[t * lddt + c] + dt_bias[c]);
  gate[idx] = scan_silu(z[t * ldz + c]);
}

extern "C" int vk_scan_prepare(float* dt, long long lddt, const float* dt_bias, const float* z, long long ldz,
                               float* gate, int num_tokens, int C, void* stream) {
  if (num_tokens <= 0) return 0;
  if (C < 1) return VK_BAD_ARGUMENT;
  const long long total = (long long)num_tokens * C;
  scan_prepare_kernel<<<(unsigned)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(dt, lddt, dt_bias, z, ldz, gate,
                                                                                       C, total);
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" long long vk_selective_scan_channel_floats(int states) { return 16LL * lanes_share(states); }

extern "C" int vk_selective_scan(const float* x, const float* dtraw, long long lddt, const float* dt_bias,
                                 const float* bmat, const float* cmat, long long ldbc, const float* a_log,
                                 const float* skip, const float* z, long long ldz, float* state,
                                 long long state_stride, const int* entry_start, const int* entry_first,
                                 const int* slots, int num_entries, int C, int N, int prepared, void* out,
                                 int out_dtype, void* stream) {
  if (num_entries <= 0) return 0;
  if (C < 1 || N < 1) return VK_BAD_ARGUMENT;
  if (N > 256) return VK_UNSUPPORTED_SIZE;
  if (state_stride < (long long)C * vk_selective_scan_channel_floats(N)) return VK_BAD_ARGUMENT;
  dim3 grid(num_entries, (C + SCAN_CHANNELS - 1) / SCAN_CHANNELS);
  if (grid.y > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
#define VK_SS(RR, TO)                                                                                               \
  selective_scan_kernel<RR, TO><<<grid, SCAN_THREADS, 0, s>>>(x, dtraw, lddt, dt_bias, bmat, cmat, ldbc, a_log, skip, \
                                                              z, ldz, state, state_stride, entry_start, entry_first, \
                                                              slots, C, N, prepared, (TO*)out)
#define VK_SS_R(TO)                       \
  switch (lanes_share(N)) {               \
    case 1: VK_SS(1, TO); break;          \
    case 2: VK_SS(2, TO); break;          \
    case 4: VK_SS(4, TO); break;          \
    case 8: VK_SS(8, TO); break;          \
    default: VK_SS(16, TO); break;        \
  }
  if (out_dtype == DT_F32) { VK_SS_R(float) }
  else if (out_dtype == DT_BF16) { VK_SS_R(bf16_t) }
  else return VK_BAD_ARGUMENT;
#undef VK_SS_R
#undef VK_SS
  VK_LAUNCH_CHECK();
  return 0;
}
