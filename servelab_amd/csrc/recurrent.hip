// Mixers whose memory is a matrix per head in a state slot: what runs between their input
// projection (float sums [T, width]) and their output projection.
//
//   lowrank_expand   z = t W2^T + b from the few columns a low-rank projection left, as a log
//                    decay (logsigmoid(z) / tau, or -exp(rate_h) softplus(z)) or plain
//   short_conv       silu of a causal convolution over time per channel (with or without a bias),
//                    the last taps - 1 inputs kept in the state slot; heads made unit vectors
//   matrix_scan      the recurrences: decay per key channel (S' = diag(a) S + k v^T), the same
//                    with the delta rule's correction (u = beta (v - S'^T k)), the matrix
//                    LSTM (scalar gates with a running maximum, a normaliser n), and the
//                    state-space form (a scalar decay per head from a step size dt, the input
//                    times dt, a skip of the token's own input)
//   head_norm_gate   a head's read-out divided by its root mean square, gain, output gate
//   projnorm_rope_store  softmax attention's q and k normed over the whole projection, rotated,
//                    k and v written to their pages
//
// Everything here is float: gates, decays and their logarithms, unit norms, the state, the
// read-out.  The activation type appears only where rows leave for a matrix product or a page.
//
// State layout: S as [head][value channel][key channel] (a column of the matrix, which one
// lane group owns, is contiguous), then what the mixer keeps besides.
#include "common.h"

__device__ __forceinline__ float softplusf_(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float logsigmoidf_(float x) { return -softplusf_(-x); }
__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }

// ------------------------------------------------------------------ low-rank expansion
// out[t][c] = f(sum_r buf[t][col + r] W2[c][r] + bias[c]);  mode 0: z, 1: logsigmoid(z) / divisor,
// 2: -exp(rates[c / per_head]) * softplus(z)
// A workgroup takes LOW_TOKENS tokens by 256 channels: a thread reads its channel's row of W2 once
// for all of them (8 tokens in a prompt's portion; 1 in a step of few tokens, which needs the blocks).
template <int LOW_TOKENS>
__global__ __launch_bounds__(256) void lowrank_expand_kernel(const float* __restrict__ buf, int stride, int col,
                                                             int rank, const float* __restrict__ w2,
                                                             const float* __restrict__ bias, int T, int C, int mode,
                                                             float divisor, const float* __restrict__ rates,
                                                             int per_head, float* __restrict__ out) {
  extern __shared__ float low[];                       // [LOW_TOKENS][rank]
  const size_t t0 = (size_t)blockIdx.x * LOW_TOKENS;
  const int nt = min(LOW_TOKENS, T - (int)t0);
  for (int i = threadIdx.x; i < LOW_TOKENS * rank; i += blockDim.x) {
    const int tt = i / rank, r = i - tt * rank;
    low[i] = tt < nt ? buf[(t0 + tt) * stride + col + r] : 0.f;
  }
  __syncthreads();
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const float* w = w2 + (size_t)c * rank;
  float z[LOW_TOKENS];
#pragma unroll
  for (int tt = 0; tt < LOW_TOKENS; ++tt) z[tt] = 0.f;
  for (int r = 0; r < rank; ++r) {
    const float wr = w[r];
#pragma unroll
    for (int tt = 0; tt < LOW_TOKENS; ++tt) z[tt] += low[tt * rank + r] * wr;
  }
  const float b = bias != nullptr ? bias[c] : 0.f;
  const float rate = mode == 2 ? -expf(rates[c / per_head]) : 0.f;
#pragma unroll
  for (int tt = 0; tt < LOW_TOKENS; ++tt) {
    if (tt >= nt) break;
    float v = z[tt] + b;
    if (mode == 1) v = logsigmoidf_(v) / divisor;
    else if (mode == 2) v = rate * softplusf_(v);
    out[(t0 + tt) * C + c] = v;
  }
}

extern "C" const char* sl_lowrank_expand(const float* buf, int stride, int col, int rank, const float* w2,
                                         const float* bias, int T, int C, int mode, float divisor,
                                         const float* rates, int heads, float* out, hipStream_t stream) {
  SL_CHECK(T >= 0 && C > 0 && rank > 0 && rank <= 1024, "lowrank_expand: sizes must be positive, rank <= 1024");
  SL_CHECK(col >= 0 && col + rank <= stride, "lowrank_expand: the columns do not fit the rows");
  SL_CHECK(mode >= 0 && mode <= 2 && heads > 0 && C % heads == 0, "lowrank_expand: unknown mode or heads");
  SL_CHECK(mode != 2 || rates != nullptr, "lowrank_expand: rates are missing");
  SL_CHECK(mode != 1 || divisor > 0.f, "lowrank_expand: the divisor must be positive");
  if (T == 0) return nullptr;
  if (T >= 32)
    lowrank_expand_kernel<8><<<dim3((T + 7) / 8, (C + 255) / 256), 256, 8 * rank * sizeof(float), stream>>>(
        buf, stride, col, rank, w2, bias, T, C, mode, divisor, rates, C / heads, out);
  else
    lowrank_expand_kernel<1><<<dim3(T, (C + 255) / 256), 256, rank * sizeof(float), stream>>>(
        buf, stride, col, rank, w2, bias, T, C, mode, divisor, rates, C / heads, out);
  return sl_launch_status();
}

// ------------------------------------------------------------------ short convolution
struct ShortConv {
  const float* buf;          // inputs of token t at buf + t * stride + col
  int stride, col, C, taps;
  const float* w;            // [C][taps], the last tap is the token's own
  const float* bias;         // [C] added before the silu, or nullptr
  float* state;              // slot s at state + s * state_stride + state_off: [taps - 1][C], oldest first
  long long state_stride;
  int state_off;
  const int* cu_q;
  const int* positions;
  const int* tok_seq;
  const int* slots;
  int unit_heads, unit_dim, scaled_heads;
  float unit_eps, scale;
  int silu;                  // 0: the convolution's sum leaves as it is
  float* out;                // [T][C]
};

// One wavefront per (token, head of the unit part | 256 other channels).
__global__ __launch_bounds__(64) void short_conv_kernel(const ShortConv a) {
  const int t = blockIdx.x, b = blockIdx.y, lane = threadIdx.x;
  int c0, n;
  if (b < a.unit_heads) {
    c0 = b * a.unit_dim;
    n = a.unit_dim;
  } else {
    c0 = a.unit_heads * a.unit_dim + (b - a.unit_heads) * 256;
    n = min(256, a.C - c0);
  }
  const int s = a.tok_seq[t];
  const int first = a.cu_q[s];
  const int i = t - first;                                  // place of the token in its step
  const bool fresh = a.positions[first] == 0;               // the sequence starts in this step
  const float* past = a.state + (size_t)a.slots[s] * a.state_stride + a.state_off;
  const int back = a.taps - 1;
  float ss = 0.f;
  float y[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int c = c0 + lane + u * 64;
    y[u] = 0.f;
    if (lane + u * 64 < n) {
      float acc = a.bias != nullptr ? a.bias[c] : 0.f;
      for (int j = 0; j < a.taps; ++j) {
        const int idx = i - back + j;                       // place in the step of the tap's input
        float x;
        if (idx >= 0) x = a.buf[(size_t)(first + idx) * a.stride + a.col + c];
        else x = fresh ? 0.f : past[(size_t)(back + idx) * a.C + c];
        acc += a.w[(size_t)c * a.taps + j] * x;
      }
      y[u] = a.silu ? acc * sigmoidf_(acc) : acc;
      ss += y[u] * y[u];
    }
  }
  float f = 1.f;
  if (b < a.unit_heads) {
    ss = wave_sum(ss);
    f = 1.f / sqrtf(ss + a.unit_eps);
    if (b < a.scaled_heads) f *= a.scale;
  }
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (lane + u * 64 < n) a.out[(size_t)t * a.C + c0 + lane + u * 64] = y[u] * f;
}

// The slot's new last inputs, after the kernel above has read the old ones: a thread per
// (sequence, channel) walks the rows oldest first; row r takes what lies len rows later, which
// is either a row it has not written yet or an input of this step.
__global__ void short_conv_state_kernel(const ShortConv a, int S) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= a.C) return;
  const int first = a.cu_q[s], len = a.cu_q[s + 1] - first;
  const bool fresh = a.positions[first] == 0;
  float* keep = a.state + (size_t)a.slots[s] * a.state_stride + a.state_off;
  const int back = a.taps - 1;
  for (int r = 0; r < back; ++r) {
    const int idx = len - back + r;
    float x;
    if (idx >= 0) x = a.buf[(size_t)(first + idx) * a.stride + a.col + c];
    else x = fresh ? 0.f : keep[(size_t)(back + idx) * a.C + c];
    keep[(size_t)r * a.C + c] = x;
  }
}

extern "C" const char* sl_short_conv(const float* buf, int stride, int col, int C, int taps, const float* w,
                                     const float* bias, float* state, long long state_stride, int state_off, const int* cu_q,
                                     const int* positions, const int* tok_seq, const int* slots, int S, int T,
                                     int write, int unit_heads, int unit_dim, float unit_eps, int scaled_heads,
                                     float scale, int silu, float* out, hipStream_t stream) {
  SL_CHECK(T >= 0 && S >= 0 && C > 0 && taps >= 1 && taps <= 64, "short_conv: sizes must be positive, taps <= 64");
  SL_CHECK(col >= 0 && col + C <= stride, "short_conv: the channels do not fit the rows");
  SL_CHECK(unit_heads >= 0 && (unit_heads == 0 || (unit_dim >= 1 && unit_dim <= 256)) &&
           (long long)unit_heads * unit_dim <= C && scaled_heads <= unit_heads,
           "short_conv: unit heads of at most 256 channels within the channels");
  SL_CHECK(state_off >= 0 && state_off + (long long)(taps - 1) * C <= state_stride,
           "short_conv: the last inputs do not fit the state slot");
  if (T == 0) return nullptr;
  const ShortConv a{buf, stride, col, C, taps, w, bias, state, state_stride, state_off, cu_q, positions, tok_seq,
                    slots, unit_heads, unit_dim, scaled_heads, unit_eps, scale, silu, out};
  const int rest = C - unit_heads * unit_dim;
  short_conv_kernel<<<dim3(T, unit_heads + (rest + 255) / 256), 64, 0, stream>>>(a);
  if (write && taps > 1) short_conv_state_kernel<<<dim3(S, (C + 255) / 256), 256, 0, stream>>>(a, S);
  return sl_launch_status();
}

// ------------------------------------------------------------------ the recurrences
struct MatrixScan {
  const float* src;          // q, k, v of token t at src + t * src_stride + {q,k,v}_col; q and k have G heads
  int src_stride, q_col, k_col, v_col;
  int H, G, D, Dv;
  const float* log_decay;    // [T][H][D] (decay and delta modes)
  float q_scale;
  const float* gates;        // delta: beta before its sigmoid at gates + t * gate_stride + beta_col + h;
  int gate_stride, i_col, f_col;   // matrix LSTM: the two gates before cap and squashing at i_col + h, f_col + h;
                             // state-space: the step size before its bias and softplus at i_col + h
  const float* rates;        // state-space, per head: dt = softplus(raw + step_bias[h]), the state keeps
  const float* step_bias;    // exp(-exp(rates[h]) dt) of itself and takes dt k v^T; the read-out adds
  const float* skip;         // skip[h] v
  float cap;
  float* state;              // slot s at state + s * state_stride: S [H][Dv][D]; matrix LSTM: then n [H][D], m [H]
  long long state_stride;
  const int* cu_q;
  const int* positions;
  const int* slots;
  int write;
  float* out;                // [T][H][Dv]
};

enum { SCAN_DECAY = 0, SCAN_DELTA = 1, SCAN_LSTM = 2, SCAN_SSD = 3 };
constexpr int SCAN_ROWS = 8;      // key channels a lane owns: channels 8 p .. 8 p + 7

// Sum over the P lanes that share a column (P a power of two, the lanes adjacent and aligned); every
// lane gets the sum.  Within 16 lanes by data-parallel moves (neighbours in a quad, the other pair of
// the quad, the mirrored half row, the mirrored row), beyond that by shuffles.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float group_sum(float v, int P) {
  if (P >= 2) v += dpp_move<0xB1>(v);          // quad_perm [1, 0, 3, 2]
  if (P >= 4) v += dpp_move<0x4E>(v);          // quad_perm [2, 3, 0, 1]
  if (P >= 8) v += dpp_move<0x141>(v);         // row_half_mirror
  if (P >= 16) v += dpp_move<0x140>(v);        // row_mirror
  for (int w = 16; w < P; w <<= 1) v += __shfl_xor(v, w, SL_WAVE);
  return v;
}
struct __attribute__((aligned(16))) scan_f4 { float v[4]; };
template <int ROWS> __device__ __forceinline__ float rows_sum(const float* x) {
  float s = (x[0] + x[1]) + (x[2] + x[3]);
  if (ROWS == 8) s += (x[4] + x[5]) + (x[6] + x[7]);
  return s;
}


// A block takes a (sequence, head, slice of value channels).  Its first four wavefronts walk the
// tokens: P lanes share a column of S (P a power of two with 8 P >= D), 256 / P columns a block, a
// lane updating its 8 rows and the P lanes of a column adding their parts of the read-out by
// butterfly.  Its other four wavefronts bring the step's tokens into LDS a chunk ahead (q, k, the
// decays after their exponential, v of the block's columns, the gates after their squashing), into
// the half of LDS that the walkers are not reading; one barrier a chunk hands the halves over.  What
// does not depend on S is done by the bringers: the matrix LSTM's running maximum and the three
// factors a token takes from it are a scan over scalars, which one of their wavefronts carries; and
// the walkers leave their read-outs in LDS, from where the bringers write a chunk's to memory.
template <int MODE, int ROWS>
__global__ __launch_bounds__(512) void matrix_scan_kernel(const MatrixScan a, int P, int CH) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int s = blockIdx.x, h = blockIdx.y, slice = blockIdx.z;
  const bool walker = threadIdx.x < 256;
  const int tid = threadIdx.x & 255;
  const int Dp = P * ROWS, cols = 256 / P;
  const int lgDp = __ffs(Dp) - 1, lgCols = __ffs(cols) - 1;
  // The matrix LSTM's normaliser n is one more column of S whose value channel is always 1: the last
  // column group of every block carries it (every block the same one) and leaves max(|n . q|, e^-m) +
  // 1e-6 where the others leave their read-outs; these are divided by it when they leave LDS.
  constexpr bool SCALAR = MODE == SCAN_LSTM || MODE == SCAN_SSD;      // one decay a head: no decays per channel in LDS
  const int vcols = MODE == SCAN_LSTM ? cols - 1 : cols;
  const int half = CH * ((SCALAR ? 2 : 3) * Dp + 2 * cols + 4);
  const int oq = 0, ok = CH * Dp, oa = 2 * CH * Dp;          // [CH][Dp] each (no decays for the matrix LSTM)
  const int ov = SCALAR ? oa : oa + CH * Dp;                  // [CH][cols]
  const int og = ov + CH * cols;                              // [CH][4] gates
  const int oo = og + CH * 4;                                 // [CH][cols] the walkers' read-outs
  const int g = h / (a.H / a.G);
  const int first = a.cu_q[s], last = a.cu_q[s + 1];
  const bool fresh = a.positions[first] == 0;
  float* slot = a.state + (size_t)a.slots[s] * a.state_stride;
  const size_t nS = (size_t)a.H * a.Dv * a.D;
  float* nrow = slot + nS + (size_t)h * a.D;
  float* mcell = slot + nS + (size_t)a.H * a.D + h;

  if (!walker) {
    float m = (MODE == SCAN_LSTM && !fresh) ? *mcell : 0.f;
    // A chunk's inputs are asked for a round ahead and wait in registers while the walkers finish the
    // chunk before: at most 8 values of q, k and the decays and 8 of v a thread (the host keeps CH
    // within that).
    float pq[8], pk[8], pd[8], pv[8], g0 = 0.f, g1 = 0.f;
    auto ask = [&](int t0, int nt) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int idx = tid + e * 256;
        pq[e] = 0.f;
        pk[e] = 0.f;
        pd[e] = 0.f;
        pv[e] = 0.f;
        if (idx < nt * Dp) {
          const int tt = idx >> lgDp, r = idx & (Dp - 1);          // (Dp and cols are powers of two)
          const size_t t = t0 + tt;
          if (r < a.D) {
            pq[e] = a.src[t * a.src_stride + a.q_col + g * a.D + r] * a.q_scale;
            pk[e] = a.src[t * a.src_stride + a.k_col + g * a.D + r];
            if (!SCALAR) pd[e] = a.log_decay[(t * a.H + h) * a.D + r];
          }
        }
        if (idx < nt * cols) {
          const int tt = idx >> lgCols, cl = idx & (cols - 1), cc = slice * vcols + cl;
          if (cl >= vcols) pv[e] = 1.f;
          else if (cc < a.Dv) pv[e] = a.src[(size_t)(t0 + tt) * a.src_stride + a.v_col + h * a.Dv + cc];
        }
      }
      if (MODE != SCAN_DECAY && tid < 64 && tid < nt) {
        const float* gr = a.gates + (size_t)(t0 + tid) * a.gate_stride;
        g0 = gr[a.i_col + h];
        if (MODE == SCAN_LSTM) g1 = gr[a.f_col + h];
      }
    };
    // the read-outs of chunk c - 2 lie in the half that round c fills: they leave for memory first
    auto flush = [&](int c, int t0) {
      if (c < 2) return;
      const float* so = lds + (c & 1) * half + oo;
      const int tf = t0 - 2 * CH, nf = min(CH, last - tf);
      for (int idx = tid; idx < nf * cols; idx += 256) {
        const int tt = idx >> lgCols, cl = idx & (cols - 1), jj = slice * vcols + cl;
        if (cl >= vcols || jj >= a.Dv) continue;
        float o = so[idx];
        if (MODE == SCAN_LSTM) o = o / so[tt * cols + cols - 1];
        a.out[((size_t)(tf + tt) * a.H + h) * a.Dv + jj] = o;
      }
    };
    ask(first, min(CH, last - first));
    for (int t0 = first, c = 0; t0 < last + CH; t0 += CH, ++c) {
      // round c brings chunk c while the walkers read chunk c - 1; the last round brings nothing
      const int nt = min(CH, last - t0);
      flush(c, t0);
      if (nt > 0) {
        float* base = lds + (c & 1) * half;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int idx = tid + e * 256;
          if (idx < nt * Dp) {
            // channel r = ROWS p + 4 u + c of a token lies at u * 4 P + 4 p + c: the 16-byte pieces that
            // the lanes of a column read together are then side by side and take every LDS bank once
            const int r = idx & (Dp - 1);
            const int at = (idx - r) + ((r & (ROWS - 1)) >> 2) * 4 * P + (r / ROWS) * 4 + (r & 3);
            base[oq + at] = pq[e];
            base[ok + at] = pk[e];
            if (!SCALAR) base[oa + at] = expf(pd[e]);
          }
          if (idx < nt * cols) base[ov + idx] = pv[e];
        }
        if (MODE == SCAN_DELTA && tid < nt) base[og + tid * 4] = sigmoidf_(g0);
        if (MODE == SCAN_SSD && tid < nt) {
          const float dt = softplusf_(g0 + a.step_bias[h]);
          base[og + tid * 4] = expf(-expf(a.rates[h]) * dt);
          base[og + tid * 4 + 1] = dt;
        }
        if (MODE == SCAN_LSTM && tid < 64) {
          // (CH is at most 16: the chunk's gates sit in the first lanes of this wavefront)
          const float ig = a.cap * tanhf(g0 / a.cap), fg = logsigmoidf_(a.cap * tanhf(g1 / a.cap));
          // the running maximum is the only chain; a lane keeps its token's two values of it and
          // takes the exponentials afterwards, all tokens at once
          float before = 0.f, top = 0.f;
          for (int tt = 0; tt < nt; ++tt) {
            const float reach = fmaxf(__shfl(fg, tt, SL_WAVE) + m, __shfl(ig, tt, SL_WAVE));
            if (tid == tt) {
              before = m;
              top = reach;
            }
            m = reach;
          }
          const float keep = expf(fg + before - top), add = expf(ig - top), floor_ = expf(-top);
          if (tid < nt) {
            base[og + tid * 4] = keep;
            base[og + tid * 4 + 1] = add;
            base[og + tid * 4 + 2] = floor_;
          }
        }
      }
      if (t0 + CH < last) ask(t0 + CH, min(CH, last - t0 - CH));
      __syncthreads();
    }
    {
      const int rounds = (last - first + CH - 1) / CH + 1;
      flush(rounds, first + rounds * CH);
    }
    if (MODE == SCAN_LSTM && a.write && slice == 0 && tid == 0) *mcell = m;
    return;
  }

  const int p = tid & (P - 1), cl = tid >> (__ffs(P) - 1);
  const bool is_n = MODE == SCAN_LSTM && cl == cols - 1;
  const int j = slice * vcols + cl;
  const bool live = is_n || j < a.Dv;
  float* col = is_n ? nrow : slot + ((size_t)h * a.Dv + (live ? j : 0)) * a.D;
  float S[ROWS];
  const float skip_h = MODE == SCAN_SSD ? a.skip[h] : 0.f;
  const int r0 = p * ROWS;
  // (a lane's values of a column are 16-byte pieces where the slot's place allows it)
  const bool whole = live && r0 + ROWS <= a.D && ((uintptr_t)(col + r0) % 16) == 0;
  if (whole && !fresh) {
#pragma unroll
    for (int u = 0; u < ROWS / 4; ++u) {
      const scan_f4 piece = ((const scan_f4*)(col + r0))[u];
#pragma unroll
      for (int c = 0; c < 4; ++c) S[4 * u + c] = piece.v[c];
    }
  }
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const int r = r0 + i;
    if (!(whole && !fresh)) S[i] = (!fresh && live && r < a.D) ? col[r] : 0.f;
  }
  __syncthreads();                        // chunk 0 is in LDS
  for (int t0 = first, c = 0; t0 < last; t0 += CH, ++c) {
    const int nt = min(CH, last - t0);
    float* base = lds + (c & 1) * half;
    const float *sq = base + oq, *sk = base + ok, *sa = base + oa, *sv = base + ov, *sg = base + og;
    float* so = base + oo;
#pragma unroll 4
    for (int tt = 0; tt < nt; ++tt) {
      float q[ROWS], k[ROWS], d[ROWS];
      {
        const scan_f4* q4 = (const scan_f4*)(sq + tt * Dp + 4 * p);
        const scan_f4* k4 = (const scan_f4*)(sk + tt * Dp + 4 * p);
        const scan_f4* d4 = (const scan_f4*)(sa + tt * Dp + 4 * p);
#pragma unroll
        for (int u = 0; u < ROWS / 4; ++u) {
          const scan_f4 qv = q4[u * P], kv = k4[u * P];
#pragma unroll
          for (int c2 = 0; c2 < 4; ++c2) {
            q[4 * u + c2] = qv.v[c2];
            k[4 * u + c2] = kv.v[c2];
          }
          if (!SCALAR) {
            const scan_f4 dv = d4[u * P];
#pragma unroll
            for (int c2 = 0; c2 < 4; ++c2) d[4 * u + c2] = dv.v[c2];
          }
        }
      }
      const float v = sv[tt * cols + cl];
      float part[ROWS];
      if (MODE == SCAN_DECAY) {
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
          S[i] = d[i] * S[i] + k[i] * v;
          part[i] = S[i] * q[i];
        }
      } else if (MODE == SCAN_DELTA) {
        // S'^T k with S' = diag(d) S, as a sum of S (d k): the products d k do not wait for S
        float dk[ROWS];
#pragma unroll
        for (int i = 0; i < ROWS; ++i) dk[i] = d[i] * k[i];
#pragma unroll
        for (int i = 0; i < ROWS; ++i) part[i] = S[i] * dk[i];
        const float seen = group_sum(rows_sum<ROWS>(part), P);
        const float u = sg[tt * 4] * (v - seen);
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
          S[i] = d[i] * S[i] + k[i] * u;
          part[i] = S[i] * q[i];
        }
      } else {
        const float keep = sg[tt * 4], av = sg[tt * 4 + 1] * v;     // (v is 1 in the column that carries n)
#pragma unroll
        for (int i = 0; i < ROWS; ++i) {
          S[i] = keep * S[i] + k[i] * av;
          part[i] = S[i] * q[i];
        }
      }
      float o = group_sum(rows_sum<ROWS>(part), P);
      // (the column that carries n leaves the divisor of its token's read-outs)
      if (MODE == SCAN_LSTM && is_n) o = fmaxf(fabsf(o), sg[tt * 4 + 2]) + 1e-6f;
      if (MODE == SCAN_SSD) o += skip_h * v;
      if (p == 0) so[tt * cols + cl] = o;
    }
    __syncthreads();                      // chunk c + 1 is in LDS, chunk c's half is free
  }
  if (a.write && (!is_n || slice == 0)) {             // (every slice carries the same n: the first writes it)
    if (whole) {
#pragma unroll
      for (int u = 0; u < ROWS / 4; ++u) {
        scan_f4 piece;
#pragma unroll
        for (int c = 0; c < 4; ++c) piece.v[c] = S[4 * u + c];
        ((scan_f4*)(col + r0))[u] = piece;
      }
    }
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int r = r0 + i;
      if (!whole && live && r < a.D) col[r] = S[i];
    }
  }
}

extern "C" const char* sl_matrix_scan(int mode, const float* src, int src_stride, int q_col, int k_col, int v_col,
                                      int H, int G, int D, int Dv, const float* log_decay, float q_scale,
                                      const float* gates, int gate_stride, int i_col, int f_col, float cap,
                                      const float* rates, const float* step_bias, const float* skip, float* state, long long state_stride, const int* cu_q, const int* positions,
                                      const int* slots, int S, int T, int write, float* out, hipStream_t stream) {
  SL_CHECK(mode >= 0 && mode <= 3, "matrix_scan: unknown mode");
  SL_CHECK(S >= 0 && T >= 0 && H > 0 && G > 0 && H % G == 0 && Dv > 0, "matrix_scan: sizes must be positive");
  SL_CHECK(D >= 1 && D <= 64 * SCAN_ROWS, "matrix_scan: at most 512 key channels a head");
  SL_CHECK(q_col >= 0 && k_col >= 0 && v_col >= 0 && q_col + G * D <= src_stride && k_col + G * D <= src_stride &&
           v_col + H * Dv <= src_stride, "matrix_scan: q, k or v do not fit the rows");
  SL_CHECK(mode == SCAN_LSTM || mode == SCAN_SSD || log_decay != nullptr, "matrix_scan: decays are missing");
  SL_CHECK(mode != SCAN_SSD || (rates != nullptr && step_bias != nullptr && skip != nullptr),
           "matrix_scan: the state-space form needs rates, step biases and skips per head");
  SL_CHECK(mode == SCAN_DECAY || (gates != nullptr && i_col >= 0 && i_col + H <= gate_stride),
           "matrix_scan: gates are missing or do not fit their rows");
  SL_CHECK(mode != SCAN_LSTM || (f_col >= 0 && f_col + H <= gate_stride && cap > 0.f),
           "matrix_scan: the forget gates do not fit their rows");
  const long long need = (long long)H * Dv * D + (mode == SCAN_LSTM ? (long long)H * D + H : 0);
  SL_CHECK(need <= state_stride, "matrix_scan: the state does not fit its slot");
  if (S == 0 || T == 0) return nullptr;
  // (A lane owning 4 key channels instead of 8 doubles the blocks of a lone prompt and halves a lane's
  // products; measured, a token takes as long: its cost is the sums across lanes, the hand-over and
  // the waits, not the products.)
  int P = 1;
  while (P * SCAN_ROWS < D) P <<= 1;
  const int cols = 256 / P, Dp = P * SCAN_ROWS;
  const int CH = min(min(16, 2048 / Dp), 8 * P);       // 8 values a thread of each kind a chunk
  const bool scalar = mode == SCAN_LSTM || mode == SCAN_SSD;
  const size_t lds = 2 * (size_t)CH * ((scalar ? 2 : 3) * Dp + 2 * cols + 4) * sizeof(float);   // two halves
  const MatrixScan a{src, src_stride, q_col, k_col, v_col, H, G, D, Dv, log_decay, q_scale, gates, gate_stride,
                     i_col, f_col, rates, step_bias, skip, cap, state, state_stride, cu_q, positions, slots, write, out};
  const int vcols = mode == SCAN_LSTM ? cols - 1 : cols;       // (the matrix LSTM's last column group carries n)
  const dim3 grid(S, H, (Dv + vcols - 1) / vcols);
  if (mode == SCAN_DECAY) matrix_scan_kernel<SCAN_DECAY, SCAN_ROWS><<<grid, 512, lds, stream>>>(a, P, CH);
  else if (mode == SCAN_DELTA) matrix_scan_kernel<SCAN_DELTA, SCAN_ROWS><<<grid, 512, lds, stream>>>(a, P, CH);
  else if (mode == SCAN_SSD) matrix_scan_kernel<SCAN_SSD, SCAN_ROWS><<<grid, 512, lds, stream>>>(a, P, CH);
  else matrix_scan_kernel<SCAN_LSTM, SCAN_ROWS><<<grid, 512, lds, stream>>>(a, P, CH);
  return sl_launch_status();
}

// ------------------------------------------------------------------ read-out: norm, gain, gate
// One wavefront per (token, head): o / sqrt(mean(o^2) + eps) * w * act(gate); act 0: sigmoid, 1: silu.
// gate_first: the gate comes before the norm, x = o * act(gate), then x / sqrt(mean(x^2) + eps) * w.
__global__ __launch_bounds__(64) void head_norm_gate_kernel(const float* __restrict__ o, int H, int Dv,
                                                            const float* __restrict__ w, int per_head, float eps,
                                                            const float* __restrict__ gate, int gate_stride,
                                                            int gate_col, int act, int gate_first,
                                                            act_t* __restrict__ out) {
  const size_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* x = o + (t * H + h) * Dv;
  const float* gr = gate + t * gate_stride + gate_col + h * Dv;
  const float* wr = w + (per_head ? h * Dv : 0);
  float ss = 0.f;
  for (int d = lane; d < Dv; d += 64) {
    float v = x[d];
    if (gate_first) {
      const float z = gr[d];
      v *= act == 0 ? sigmoidf_(z) : z * sigmoidf_(z);
    }
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(wave_sum(ss) / (float)Dv + eps);
  for (int d = lane; d < Dv; d += 64) {
    const float z = gr[d];
    const float gv = act == 0 ? sigmoidf_(z) : z * sigmoidf_(z);
    out[(t * H + h) * Dv + d] = from_f<act_t>(gate_first ? (x[d] * gv) * inv * wr[d] : x[d] * inv * wr[d] * gv);
  }
}

extern "C" const char* sl_head_norm_gate(const float* o, int T, int H, int Dv, const float* w, int per_head,
                                         float eps, const float* gate, int gate_stride, int gate_col, int act,
                                         int gate_first, void* out, hipStream_t stream) {
  SL_CHECK(T >= 0 && H > 0 && Dv > 0, "head_norm_gate: sizes must be positive");
  SL_CHECK(gate_col >= 0 && gate_col + H * Dv <= gate_stride, "head_norm_gate: the gates do not fit their rows");
  SL_CHECK(act == 0 || act == 1, "head_norm_gate: the gate is sigmoid (0) or silu (1)");
  if (T == 0) return nullptr;
  head_norm_gate_kernel<<<dim3(T, H), 64, 0, stream>>>(o, H, Dv, w, per_head, eps, gate, gate_stride, gate_col,
                                                       act, gate_first, (act_t*)out);
  return sl_launch_status();
}

// ------------------------------------------------------------------ softmax attention's q, k, v
// buf row: q [H][D], k [G][D], v [G][Dv] (float).  q and k are divided by the root mean square of
// all their heads together and multiplied by a gain of that size (no gains: no norm), then the first `rot` channels
// of every head turn in halves (channel i with i + rot / 2, angle of cos/sin column i).  q leaves
// in the activation type; k and v go to the token's place in the pages.  The values lie at column
// v_col of the row (behind k: (H + G) D; at H D the values are the keys as the projection left
// them, before norm and rotation).  One block per token.
// With taps given, the row's first conv_C channels first pass a short causal convolution over time
// (no bias, no activation; the sums of short_conv_kernel in the same order): the block leaves its
// token's sums in LDS and goes on from there, so the convolved rows never reach memory.  The
// state's new last inputs are written by short_conv_state_kernel, launched behind this one.
__global__ void projnorm_rope_store_kernel(const float* __restrict__ buf, int stride, int H, int G, int D, int Dv,
                                           const float* __restrict__ qw, const float* __restrict__ kw, float eps,
                                           int rot, const float* __restrict__ cosv, const float* __restrict__ sinv,
                                           const int* __restrict__ slots, act_t* __restrict__ kc,
                                           act_t* __restrict__ vc, int page, act_t* __restrict__ q_out,
                                           int v_col, const ShortConv cv) {
  __shared__ float scratch[16];
  extern __shared__ float convolved[];       // [cv.C] when a convolution comes first
  const size_t t = blockIdx.x;
  const float* row = buf + t * stride;
  if (cv.w != nullptr) {
    const int s = cv.tok_seq[t];
    const int first = cv.cu_q[s];
    const int i = (int)t - first;
    const bool fresh = cv.positions[first] == 0;
    const float* past = cv.state + (size_t)cv.slots[s] * cv.state_stride + cv.state_off;
    const int back = cv.taps - 1;
    for (int c = threadIdx.x; c < cv.C; c += blockDim.x) {
      float acc = 0.f;
      for (int j = 0; j < cv.taps; ++j) {
        const int idx = i - back + j;
        float x;
        if (idx >= 0) x = buf[(size_t)(first + idx) * stride + c];
        else x = fresh ? 0.f : past[(size_t)(back + idx) * cv.C + c];
        acc += cv.w[(size_t)c * cv.taps + j] * x;
      }
      convolved[c] = acc;
    }
    __syncthreads();
    row = convolved;
  }
  const int nq = H * D, nk = G * D, nv = G * Dv;
  float sq = 0.f, sk = 0.f;
  const bool normed = qw != nullptr;
  float iq = 1.f, ik = 1.f;
  if (normed) {
    for (int e = threadIdx.x; e < nq; e += blockDim.x) sq += row[e] * row[e];
    for (int e = threadIdx.x; e < nk; e += blockDim.x) sk += row[nq + e] * row[nq + e];
    iq = 1.f / sqrtf(block_sum(sq, scratch) / (float)nq + eps);
    ik = 1.f / sqrtf(block_sum(sk, scratch) / (float)nk + eps);
  }
  const int half = rot / 2;
  const float* cs = cosv != nullptr ? cosv + t * half : nullptr;
  const float* sn = sinv != nullptr ? sinv + t * half : nullptr;
  const int slot = slots != nullptr ? slots[t] : 0;
  const size_t pg = slot / page, off = slot % page;
  for (int e = threadIdx.x; e < nq + nk; e += blockDim.x) {
    const bool is_q = e < nq;
    const int el = is_q ? e : e - nq;
    const float* x = is_q ? row : row + nq;
    const float* w = is_q ? qw : kw;
    const float inv = is_q ? iq : ik;
    const int d = el % D;
    float v = normed ? x[el] * inv * w[el] : x[el];
    if (d < rot) {
      const int i = d < half ? d : d - half;
      const int partner = d < half ? el + half : el - half;
      const float o = normed ? x[partner] * inv * w[partner] : x[partner];
      v = d < half ? v * cs[i] - o * sn[i] : v * cs[i] + o * sn[i];
    }
    if (is_q) q_out[t * nq + el] = from_f<act_t>(v);
    else if (slots != nullptr) kc[((pg * G + el / D) * page + off) * D + d] = from_f<act_t>(v);
  }
  if (slots != nullptr)
    for (int e = threadIdx.x; e < nv; e += blockDim.x)
      vc[((pg * G + e / Dv) * Dv + e % Dv) * page + off] = from_f<act_t>(row[v_col + e]);
}

// The same without a norm over the projection, where nothing ties a token's heads together: one
// wavefront per (token, head of q, k or v), so that a step of few tokens still fills the chip
// and the convolution's loads (a head's channels over the taps, and their partners' for the
// rotation) are all in flight together.  The sums run in the order of the kernel above.
__global__ __launch_bounds__(64) void rope_store_heads_kernel(const float* __restrict__ buf, int stride, int H, int G, int D,
                                                              int Dv, int rot, const float* __restrict__ cosv,
                                                              const float* __restrict__ sinv,
                                                              const int* __restrict__ slots, act_t* __restrict__ kc,
                                                              act_t* __restrict__ vc, int page,
                                                              act_t* __restrict__ q_out, int v_col, const ShortConv cv) {
  const size_t t = blockIdx.x;
  const int hb = blockIdx.y, lane = threadIdx.x;
  const float* row = buf + t * stride;
  int first = 0, i = 0, back = 0;
  bool fresh = true;
  const float* past = nullptr;
  if (cv.w != nullptr) {
    const int s = cv.tok_seq[t];
    first = cv.cu_q[s];
    i = (int)t - first;
    fresh = cv.positions[first] == 0;
    past = cv.state + (size_t)cv.slots[s] * cv.state_stride + cv.state_off;
    back = cv.taps - 1;
  }
  auto value = [&](int c) -> float {
    if (cv.w == nullptr) return row[c];
    float acc = 0.f;
    for (int j = 0; j < cv.taps; ++j) {
      const int idx = i - back + j;
      float x;
      if (idx >= 0) x = buf[(size_t)(first + idx) * stride + c];
      else x = fresh ? 0.f : past[(size_t)(back + idx) * cv.C + c];
      acc += cv.w[(size_t)c * cv.taps + j] * x;
    }
    return acc;
  };
  const int slot = slots != nullptr ? slots[t] : 0;
  const size_t pg = slot / page, off = slot % page;
  if (hb >= H + G) {                                   // a head of v
    if (slots == nullptr) return;
    const int g = hb - H - G;
    for (int d = lane; d < Dv; d += 64)
      vc[((pg * G + g) * Dv + d) * page + off] = from_f<act_t>(value(v_col + g * Dv + d));
    return;
  }
  const bool is_q = hb < H;
  if (!is_q && slots == nullptr) return;
  const int base = hb * D;                             // (k heads follow the q heads in the row)
  const int half = rot / 2;
  for (int d = lane; d < D; d += 64) {
    float v = value(base + d);
    if (d < rot) {
      const int p = d < half ? d : d - half;
      const float o = value(base + (d < half ? d + half : d - half));
      const float cs = cosv[t * half + p], sn = sinv[t * half + p];
      v = d < half ? v * cs - o * sn : v * cs + o * sn;
    }
    if (is_q) q_out[t * (size_t)(H * D) + base + d] = from_f<act_t>(v);
    else kc[((pg * G + (hb - H)) * page + off) * D + d] = from_f<act_t>(v);
  }
}

extern "C" const char* sl_projnorm_rope_store(const float* buf, int stride, int T, int H, int G, int D, int Dv,
                                              const float* qw, const float* kw, float eps, int rot,
                                              const float* cosv, const float* sinv, const int* slots, void* kc,
                                              void* vc, int page, void* q_out, int v_col,
                                              const float* taps_w, int taps, int conv_C, float* state,
                                              long long state_stride, int state_off, const int* cu_q,
                                              const int* positions, const int* tok_seq, const int* state_slots,
                                              int S, int write_state, hipStream_t stream) {
  SL_CHECK(T >= 0 && H > 0 && G > 0 && D > 0 && Dv > 0 && page > 0, "projnorm_rope_store: sizes must be positive");
  SL_CHECK((long long)(H + G) * D <= stride && v_col >= 0 && v_col + (long long)G * Dv <= stride,
           "projnorm_rope_store: q, k and v do not fit the rows");
  SL_CHECK(rot >= 0 && rot % 2 == 0 && rot <= D, "projnorm_rope_store: the rotated width must be even and within a head");
  SL_CHECK(rot == 0 || (cosv != nullptr && sinv != nullptr), "projnorm_rope_store: cos and sin are missing");
  SL_CHECK((qw == nullptr) == (kw == nullptr), "projnorm_rope_store: both gains or neither");
  SL_CHECK(slots == nullptr || (kc != nullptr && vc != nullptr), "projnorm_rope_store: pages are missing");
  ShortConv cv{};
  size_t lds = 0;
  if (taps_w != nullptr) {
    SL_CHECK(taps >= 1 && taps <= 64 && conv_C > 0 && conv_C <= stride && conv_C <= 12288,
             "projnorm_rope_store: a convolution of 1..64 taps over at most 12,288 channels within the rows");
    SL_CHECK(v_col + (long long)G * Dv <= conv_C, "projnorm_rope_store: q, k and v must all pass the convolution");
    SL_CHECK(cu_q != nullptr && positions != nullptr && tok_seq != nullptr && state_slots != nullptr && state != nullptr,
             "projnorm_rope_store: the convolution needs the step's sequences and a state");
    SL_CHECK(state_off >= 0 && state_off + (long long)(taps - 1) * conv_C <= state_stride,
             "projnorm_rope_store: the last inputs do not fit the state slot");
    cv = ShortConv{buf, stride, 0, conv_C, taps, taps_w, nullptr, state, state_stride, state_off, cu_q, positions,
                   tok_seq, state_slots, 0, 0, 0, 0.f, 1.f, 0, nullptr};
    lds = (size_t)conv_C * sizeof(float);
  }
  if (T == 0) return nullptr;
  // (few tokens: a wavefront per head fills the chip; many: a block per token computes every channel's
  // convolution once, where the heads' wavefronts compute the rotated ones twice: 2,048 tokens of 20 heads
  // of 128 channels, 4 taps: 32 against 50 us; 8 tokens: 28 against 9 us)
  if (qw == nullptr && H + 2 * G <= 65535 && T < 512)
    rope_store_heads_kernel<<<dim3(T, H + 2 * G), 64, 0, stream>>>(buf, stride, H, G, D, Dv, rot, cosv, sinv, slots,
                                                                   (act_t*)kc, (act_t*)vc, page, (act_t*)q_out, v_col, cv);
  else   // (a step of few tokens has few blocks: wider ones shorten each block's loops over the row)
    projnorm_rope_store_kernel<<<T, T <= 64 ? 1024 : 256, lds, stream>>>(buf, stride, H, G, D, Dv, qw, kw, eps, rot, cosv, sinv, slots,
                                                        (act_t*)kc, (act_t*)vc, page, (act_t*)q_out, v_col, cv);
  if (taps_w != nullptr && write_state && taps > 1)
    short_conv_state_kernel<<<dim3(S, (conv_C + 255) / 256), 256, 0, stream>>>(cv, S);
  return sl_launch_status();
}
