// Attention over the paged cache with the extras that some designs put around
// the softmax, each switched by a parameter of the call:
//   * keys and values of different widths (Dk, Dv); values read from the value
//     pages, or, when no values are stored, from the first Dv channels of the
//     key rows (a cached latent that serves as key and as value);
//   * a window that also keeps the first tokens: the query at position i of its
//     sequence sees key j <= i when i - j < window or j < keep_first;
//   * capped scores: the scaled score s becomes c tanh(s / c);
//   * a distance bias: slope_h * (i - j) is taken off the scaled score;
//   * a sink: exp(sink_h) enters the softmax's denominator once, without a key
//     or a value;
//   * an output gate: the head's output is multiplied by sigmoid(gate[t, h]).
// Scores, weights, the running maximum and sum and the output sums are float
// in both builds; q, keys and values arrive in the activation type.
//
// A workgroup of four wavefronts owns 16 columns, a column being a (token,
// query head) pair of one sequence and one kv head, and walks the blocks of KB
// keys that any of its columns sees; a block is staged in LDS as floats once
// for all columns.  16 lanes share a column: they split a block's keys for the
// scores and the value channels for the output.  A prompt portion sees itself
// through the cache (its keys are written first), so a decoded token is a
// portion of one token whose 16 columns are the heads of its group.  The blocks
// of a tile may be cut into shares (few tokens over many keys); the shares
// leave unnormalised sums, and a second kernel merges them.
//
// The file also holds what runs before such attention: the per-head RMS norm of
// q and k with the write of k and (mixed) v into their pages, and the write of a
// latent row with its rotated part.
#include "window_attention.h"

constexpr int WA_COLS = 16;
constexpr int WA_THREADS = 256;

template <int KB, int NJ>
__global__ __launch_bounds__(WA_THREADS) void window_attention_kernel(const WindowAttention a) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int Dk = a.Dk, Dv = a.Dv, page = a.page, nkv = a.nkv;
  const int DkP = (Dk + 3) & ~3, KS = DkP + 4, VS = Dv + 1;
  float* qs = lds;                                   // [WA_COLS][DkP]
  float* ks = qs + WA_COLS * DkP;                    // [KB][KS]
  float* vs = ks + KB * KS;                          // [KB][VS] (only with value pages)
  float* ps = vs + (a.vc != nullptr ? KB * VS : 0);  // [WA_COLS][KB]
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int sub = lane & 15, col = 4 * wave + (lane >> 4);
  const int seq = blockIdx.z, kvh = blockIdx.y;
  const int g = a.nh / nkv;
  const int q0 = a.cu_q[seq], qlen = a.cu_q[seq + 1] - q0;
  const int ncols = qlen * g;
  const int tile = blockIdx.x / a.nsplit, share = blockIdx.x % a.nsplit;
  const int c0 = tile * WA_COLS;
  if (c0 >= ncols) return;
  const int pos0 = a.positions[q0];
  const int* table = a.tables + (size_t)seq * a.max_pages;

  const int c = c0 + col;
  const bool live = c < ncols;
  const int tok = live ? c / g : 0, head = kvh * g + (live ? c % g : 0);
  const int pos_c = live ? pos0 + tok : -1;
  const int lo_c = a.window > 0 && pos_c - a.window + 1 > 0 ? pos_c - a.window + 1 : 0;
  const float slope = a.slopes != nullptr ? a.slopes[head] : 0.f;
  const int tok_first = c0 / g;
  const int c_last = c0 + WA_COLS - 1 < ncols - 1 ? c0 + WA_COLS - 1 : ncols - 1;
  const int kmax = pos0 + c_last / g;
  int kmin = 0;
  if (a.window > 0 && pos0 + tok_first - a.window + 1 > 0) kmin = pos0 + tok_first - a.window + 1;
  const int keep = a.keep_first < kmin ? a.keep_first : kmin;      // keys [0, keep) and [kmin, kmax]
  // blocks [0, nA) hold the kept first keys, blocks [firstB, firstB + nB) the window
  const int nA = keep > 0 ? (keep - 1) / KB + 1 : 0;
  int firstB = kmin / KB;
  if (firstB < nA) firstB = nA;
  const int nB = kmax / KB - firstB + 1 > 0 ? kmax / KB - firstB + 1 : 0;
  const int nblk = nA + nB;
  const int i0 = (int)((long long)nblk * share / a.nsplit);
  const int i1 = (int)((long long)nblk * (share + 1) / a.nsplit);

  for (int idx = t; idx < WA_COLS * DkP; idx += WA_THREADS) {
    const int cc = c0 + idx / DkP, d = idx % DkP;
    qs[idx] = cc < ncols && d < Dk
        ? to_f(a.q[(size_t)(q0 + cc / g) * a.q_stride + (size_t)(kvh * g + cc % g) * Dk + d]) : 0.f;
  }

  float m = -INFINITY, l = 0.f;
  float acc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) acc[j] = 0.f;

  for (int i = i0; i < i1; ++i) {
    const int kbase = (i < nA ? i : firstB + (i - nA)) * KB;
    __syncthreads();                                 // the last block's readers are done (and qs is written)
    for (int idx = t; idx < KB * DkP; idx += WA_THREADS) {
      const int kk = idx / DkP, d = idx % DkP, key = kbase + kk;
      float v = 0.f;
      if (d < Dk && key <= kmax && (key >= kmin || key < keep)) {
        const int pg = table[key / page];
        v = to_f(a.kc[(((size_t)pg * nkv + kvh) * page + key % page) * Dk + d]);
      }
      ks[kk * KS + d] = v;
    }
    if (a.vc != nullptr) {
      for (int idx = t; idx < KB * Dv; idx += WA_THREADS) {
        const int kk = idx % KB, d = idx / KB, key = kbase + kk;
        float v = 0.f;
        if (key <= kmax && (key >= kmin || key < keep)) {
          const int pg = table[key / page];
          v = to_f(a.vc[(((size_t)pg * nkv + kvh) * Dv + d) * page + key % page]);
        }
        vs[kk * VS + d] = v;
      }
    }
    __syncthreads();
    float sc[KB / 16];
#pragma unroll
    for (int r = 0; r < KB / 16; ++r) sc[r] = 0.f;
    const float* qrow = qs + col * DkP;
    for (int d = 0; d < DkP; d += 4) {
      const float4 q4 = *(const float4*)(qrow + d);
#pragma unroll
      for (int r = 0; r < KB / 16; ++r) {
        const float4 k4 = *(const float4*)(ks + (sub + 16 * r) * KS + d);
        sc[r] += q4.x * k4.x + q4.y * k4.y + q4.z * k4.z + q4.w * k4.w;
      }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int r = 0; r < KB / 16; ++r) {
      const int key = kbase + sub + 16 * r;
      const bool sees = key <= pos_c && (key >= lo_c || key < a.keep_first);
      float sv = sc[r] * a.scale;
      if (a.softcap > 0.f) sv = a.softcap * tanhf(sv / a.softcap);
      sc[r] = sees ? sv - slope * (float)(pos_c - key) : -INFINITY;
      mx = fmaxf(mx, sc[r]);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    const float mn = fmaxf(m, mx);
    // a column that has seen no key yet keeps m = -inf: nothing to rescale, nothing to add
    const float alpha = mn == -INFINITY ? 1.f : expf(m - mn);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < KB / 16; ++r) {
      const float pr = sc[r] == -INFINITY ? 0.f : expf(sc[r] - mn);
      psum += pr;
      ps[col * KB + sub + 16 * r] = pr;
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) psum += __shfl_xor(psum, o, 64);
    l = l * alpha + psum;
    m = mn;
    __syncthreads();                                 // ps is complete
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[j] *= alpha;
    const float* prow = ps + col * KB;
    const float* vals = a.vc != nullptr ? vs : ks;
    const int stride = a.vc != nullptr ? VS : KS;
    for (int kk = 0; kk < KB; ++kk) {
      const float pk = prow[kk];
      const float* vrow = vals + kk * stride + sub;
#pragma unroll
      for (int j = 0; j < NJ; ++j)
        if (16 * j + sub < Dv) acc[j] += pk * vrow[16 * j];
    }
  }
  if (!live) return;
  const size_t row = (size_t)(q0 + tok) * a.nh + head;
  if (a.nsplit > 1) {
    float* po = a.part_o + (row * a.nsplit + share) * Dv;
#pragma unroll
    for (int j = 0; j < NJ; ++j)
      if (16 * j + sub < Dv) po[16 * j + sub] = acc[j];
    if (sub == 0) {
      a.part_ml[(row * a.nsplit + share) * 2] = m;
      a.part_ml[(row * a.nsplit + share) * 2 + 1] = l;
    }
    return;
  }
  // every query sees itself, so m is finite here
  float top = m, extra = 0.f;
  if (a.sinks != nullptr) {
    const float sink = a.sinks[head];
    top = fmaxf(m, sink);
    extra = expf(sink - top);
  }
  const float w = expf(m - top);
  float f = w / (l * w + extra);
  if (a.gate != nullptr) f *= sigmoidf_(to_f(a.gate[(size_t)(q0 + tok) * a.gate_stride + head]));
  act_t* o = a.out + row * Dv;
#pragma unroll
  for (int j = 0; j < NJ; ++j)
    if (16 * j + sub < Dv) o[16 * j + sub] = from_f<act_t>(acc[j] * f);
}

template <int KB>
static const char* launch_window_attention(const WindowAttention& a, dim3 grid, size_t bytes,
                                           hipStream_t stream) {
  const int nj = (a.Dv + 15) / 16;
#define WA_LAUNCH(NJ)                                                                              \
  do {                                                                                             \
    if (bytes > 48 * 1024) {                                                                       \
      hipError_t e = hipFuncSetAttribute((const void*)window_attention_kernel<KB, NJ>,             \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);  \
      if (e != hipSuccess) return hipGetErrorString(e);                                            \
    }                                                                                              \
    window_attention_kernel<KB, NJ><<<grid, WA_THREADS, bytes, stream>>>(a);                       \
  } while (0)
  if (nj <= 2) WA_LAUNCH(2);
  else if (nj <= 4) WA_LAUNCH(4);
  else if (nj <= 8) WA_LAUNCH(8);
  else if (nj <= 16) WA_LAUNCH(16);
  else WA_LAUNCH(32);
#undef WA_LAUNCH
  return sl_launch_status();
}

// Sequences [0, num_seqs) of the batch, at most max_q_len tokens each.
extern "C" const char* sl_window_attention(
    const void* q, int q_stride, const void* kc, const void* vc, const int* tables, int max_pages,
    const int* cu_q, const int* positions, int num_seqs, int max_q_len, int num_tokens, int nh,
    int nkv, int Dk, int Dv, int page, float scale, float softcap, int window, int keep_first, const float* slopes,
    const float* sinks, const void* gate, int gate_stride, void* out, int nsplit, float* part_o,
    float* part_ml, hipStream_t stream) {
  SL_CHECK(num_seqs >= 0 && max_q_len >= 1 && nh > 0 && nkv > 0 && nh % nkv == 0,
           "window attention: heads must be a positive multiple of kv heads");
  SL_CHECK(Dk > 0 && Dv > 0 && Dv <= 512, "window attention: value width must be in 1..512");
  SL_CHECK(vc != nullptr || Dv <= Dk, "window attention: values read from key rows cannot be wider than a key");
  SL_CHECK(page == 16 || page == 32 || page == 64, "window attention: page size must be 16, 32 or 64");
  SL_CHECK(nkv <= 65535 && num_seqs <= 65535, "window attention: grid too large");
  SL_CHECK(window >= 0 && keep_first >= 0 && softcap >= 0.f, "window attention: window, keep_first and the cap must be >= 0");
  SL_CHECK(nsplit >= 1 && nsplit <= 64, "window attention: 1..64 shares of the keys");
  SL_CHECK(nsplit == 1 || (part_o != nullptr && part_ml != nullptr),
           "window attention: shares of the keys need the partial buffers");
  SL_CHECK(gate == nullptr || gate_stride >= nh, "window attention: gate rows are shorter than the heads");
  if (num_seqs == 0 || num_tokens == 0) return nullptr;
  const long long cols = (long long)max_q_len * (nh / nkv);
  const long long tiles = (cols + WA_COLS - 1) / WA_COLS;
  SL_CHECK(tiles * nsplit <= 1 << 30, "window attention: too many column tiles");
  const WindowAttention a{(const act_t*)q, q_stride, (const act_t*)kc, (const act_t*)vc, tables, max_pages,
                          cu_q, positions, nh, nkv, Dk, Dv, page, scale, softcap, window, keep_first, slopes, sinks,
                          (const act_t*)gate, gate_stride, (act_t*)out, nsplit, part_o, part_ml};
  const dim3 grid((unsigned)(tiles * nsplit), nkv, num_seqs);
  const int DkP = (Dk + 3) & ~3;
  auto need = [&](int KB) {
    return sizeof(float) * ((size_t)WA_COLS * DkP + (size_t)KB * (DkP + 4) +
                            (vc != nullptr ? (size_t)KB * (Dv + 1) : 0) + (size_t)WA_COLS * KB);
  };
  const char* e;
  if (need(32) <= 64 * 1024) e = launch_window_attention<32>(a, grid, need(32), stream);
  else {
    SL_CHECK(need(16) <= 160 * 1024, "window attention: the heads are too wide for LDS");
    e = launch_window_attention<16>(a, grid, need(16), stream);
  }
  if (e || nsplit == 1) return e;
  window_attention_combine_kernel<<<dim3(num_tokens, nh, (Dv + 63) / 64), 64, 0, stream>>>(
      part_o, part_ml, nsplit, nh, Dv, sinks, (const act_t*)gate, gate_stride, (act_t*)out);
  return sl_launch_status();
}

// ---------------------------------------------------------------------------
// Before the attention: q and k heads divided by their root mean square (over
// the head's channels, eps inside the root) and multiplied by a gain shared by
// all heads; k and v written to their cache rows; v optionally mixed with the
// values another layer made for the same tokens:  v <- (1 - lambda) v + lambda v_first.
// buf row t holds [q: nh * Dk | k: nkv * Dk | v: nkv * Dv | ...]; q is normed in
// place, k and v only go to the cache.  One wavefront per (token, head).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void headnorm_store_kernel(
    act_t* __restrict__ buf, int stride, int nh, int nkv, int Dk, int Dv,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const act_t* __restrict__ v_first, int v_first_stride, float lambda,
    const int* __restrict__ slots, act_t* __restrict__ kc, act_t* __restrict__ vc, int page) {
  const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  act_t* row = buf + (size_t)t * stride;
  if (unit < nh + nkv) {
    const bool is_q = unit < nh;
    const float* gain = is_q ? q_gain : k_gain;
    act_t* x = row + (size_t)unit * Dk;               // (k heads follow the q heads)
    if (is_q && gain == nullptr) return;
    float ss = 0.f;
    for (int d = lane; d < Dk; d += 64) {
      const float v = to_f(x[d]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = gain != nullptr ? 1.f / sqrtf(ss / (float)Dk + eps) : 1.f;
    if (is_q) {
      for (int d = lane; d < Dk; d += 64) x[d] = from_f<act_t>(to_f(x[d]) * inv * gain[d]);
      return;
    }
    if (slots == nullptr) return;
    const int slot = slots[t], kv = unit - nh;
    act_t* dst = kc + (((size_t)(slot / page) * nkv + kv) * page + slot % page) * Dk;
    for (int d = lane; d < Dk; d += 64)
      dst[d] = from_f<act_t>(to_f(x[d]) * inv * (gain != nullptr ? gain[d] : 1.f));
    return;
  }
  if (slots == nullptr) return;
  const int kv = unit - nh - nkv, slot = slots[t];
  const act_t* x = row + (size_t)(nh + nkv) * Dk + (size_t)kv * Dv;
  const act_t* f = v_first != nullptr ? v_first + (size_t)t * v_first_stride + (size_t)kv * Dv : nullptr;
  act_t* dst = vc + ((size_t)(slot / page) * nkv + kv) * Dv * page + slot % page;
  for (int d = lane; d < Dv; d += 64) {
    float v = to_f(x[d]);
    if (f != nullptr) v = (1.f - lambda) * v + lambda * to_f(f[d]);
    dst[(size_t)d * page] = from_f<act_t>(v);
  }
}

extern "C" const char* sl_headnorm_store(void* buf, int stride, int T, int nh, int nkv, int Dk, int Dv,
                                         const float* q_gain, const float* k_gain, float eps,
                                         const void* v_first, int v_first_stride, float lambda,
                                         const int* slots, void* kc, void* vc, int page,
                                         hipStream_t stream) {
  SL_CHECK(T >= 0 && nh > 0 && nkv > 0 && Dk > 0 && Dv > 0, "headnorm_store: sizes must be positive");
  SL_CHECK(stride >= (nh + nkv) * Dk + nkv * Dv, "headnorm_store: rows are shorter than q, k and v");
  SL_CHECK(nh + 2 * nkv <= 65535, "headnorm_store: too many heads");
  SL_CHECK(slots == nullptr || (kc != nullptr && vc != nullptr && page > 0),
           "headnorm_store: a cache write needs the pages");
  SL_CHECK(v_first == nullptr || v_first_stride >= nkv * Dv, "headnorm_store: rows of the other values are too short");
  if (T == 0) return nullptr;
  headnorm_store_kernel<<<dim3(T, nh + 2 * nkv), 64, 0, stream>>>(
      (act_t*)buf, stride, nh, nkv, Dk, Dv, q_gain, k_gain, eps, (const act_t*)v_first, v_first_stride,
      lambda, slots, (act_t*)kc, (act_t*)vc, page);
  return sl_launch_status();
}

// ---------------------------------------------------------------------------
// A latent row and its rotated part.  The query heads of token t lie in qbuf row t
// and, in dbuf row t (which may be the same rows) from column down_off on,
// [C channels | R channels]: the first C are divided by their root mean square
// and multiplied by a gain, and are the latent; of the last R the first `rot`
// are rotated by the token's angles (pair i, i + rot / 2), the rest pass.  Both
// go to the key row of the token's cache slot ([C | R], one kv head).  The last
// R channels of each of the nh query heads (head h at column h * (D + R) + D)
// are rotated the same way and written to q_out[t][h][C .. C + R).
// One wavefront per (token, unit): unit 0 the latent row, unit 1 + h head h.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64) void latent_store_kernel(
    const act_t* __restrict__ qbuf, int q_stride, const act_t* __restrict__ dbuf, int stride, int nh, int D, int R,
    int C, int down_off, int rot, const float* __restrict__ gain, float eps, const float* __restrict__ cosv,
    const float* __restrict__ sinv, const int* __restrict__ slots, act_t* __restrict__ kc, int page,
    act_t* __restrict__ q_out) {
  const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
  const act_t* row = dbuf + (size_t)t * stride;
  const int half = rot / 2;
  const act_t* src;
  act_t* dst;
  if (unit == 0) {
    if (slots == nullptr) return;
    const int slot = slots[t];
    act_t* krow = kc + (size_t)slot * (C + R);         // (one kv head: a page's rows are consecutive)
    const act_t* x = row + down_off;
    float ss = 0.f;
    for (int d = lane; d < C; d += 64) {
      const float v = to_f(x[d]);
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)C + eps);
    for (int d = lane; d < C; d += 64) krow[d] = from_f<act_t>(to_f(x[d]) * inv * gain[d]);
    src = x + C;
    dst = krow + C;
  } else {
    const int h = unit - 1;
    src = qbuf + (size_t)t * q_stride + (size_t)h * (D + R) + D;
    dst = q_out + ((size_t)t * nh + h) * (C + R) + C;
  }
  for (int i = lane; i < half; i += 64) {
    const float c = cosv[(size_t)t * half + i], s = sinv[(size_t)t * half + i];
    const float u = to_f(src[i]), v = to_f(src[i + half]);
    dst[i] = from_f<act_t>(u * c - v * s);
    dst[i + half] = from_f<act_t>(v * c + u * s);
  }
  for (int d = rot + lane; d < R; d += 64) dst[d] = src[d];
}

extern "C" const char* sl_latent_store(const void* qbuf, int q_stride, const void* buf, int stride, int T, int nh,
                                       int D, int R, int C,
                                       int down_off, int rot, const float* gain, float eps,
                                       const float* cosv, const float* sinv, const int* slots, void* kc,
                                       int page, void* q_out, hipStream_t stream) {
  SL_CHECK(T >= 0 && nh > 0 && D > 0 && R > 0 && C > 0, "latent_store: sizes must be positive");
  SL_CHECK(rot % 2 == 0 && rot >= 0 && rot <= R, "latent_store: the rotated width must be even and within R");
  SL_CHECK(down_off >= 0 && stride >= down_off + C + R && q_stride >= nh * (D + R) &&
           (qbuf != buf || down_off >= nh * (D + R)), "latent_store: rows are too short");
  SL_CHECK(nh + 1 <= 65535, "latent_store: too many heads");
  SL_CHECK(rot == 0 || (cosv != nullptr && sinv != nullptr), "latent_store: a rotation needs its tables");
  SL_CHECK(gain != nullptr && q_out != nullptr, "latent_store: gain and q_out are required");
  SL_CHECK(slots == nullptr || (kc != nullptr && page > 0), "latent_store: a cache write needs the pages");
  if (T == 0) return nullptr;
  latent_store_kernel<<<dim3(T, nh + 1), 64, 0, stream>>>(
      (const act_t*)qbuf, q_stride, (const act_t*)buf, stride, nh, D, R, C, down_off, rot, gain, eps, cosv, sinv,
      slots, (act_t*)kc, page, (act_t*)q_out);
  return sl_launch_status();
}

// ---------------------------------------------------------------------------
// The RMS norm of a slice of columns: out[t][c] = x[t][col + c] * rsqrt(mean_c x^2 + eps) * gain[c],
// sums in float.  One block per token: a thread asks for all its values at once (up to SLICE_KEEP of
// them stay in registers, so the row makes one trip from memory) and the gains with them.
// ---------------------------------------------------------------------------
constexpr int SLICE_KEEP = 8;
__global__ __launch_bounds__(256) void slice_rmsnorm_kernel(const act_t* __restrict__ buf, int stride, int col, int n,
                                                            const float* __restrict__ gain, float eps,
                                                            act_t* __restrict__ out) {
  __shared__ float scratch[16];
  const size_t t = blockIdx.x;
  const act_t* x = buf + t * stride + col;
  float keep[SLICE_KEEP], g[SLICE_KEEP];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < SLICE_KEEP; ++u) {
    const int d = threadIdx.x + u * 256;
    keep[u] = d < n ? to_f(x[d]) : 0.f;
    g[u] = d < n ? gain[d] : 0.f;
  }
#pragma unroll
  for (int u = 0; u < SLICE_KEEP; ++u) ss += keep[u] * keep[u];
  for (int d = threadIdx.x + SLICE_KEEP * 256; d < n; d += 256) {
    const float v = to_f(x[d]);
    ss += v * v;
  }
  const float inv = 1.f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
#pragma unroll
  for (int u = 0; u < SLICE_KEEP; ++u) {
    const int d = threadIdx.x + u * 256;
    if (d < n) out[t * n + d] = from_f<act_t>(keep[u] * inv * g[u]);
  }
  for (int d = threadIdx.x + SLICE_KEEP * 256; d < n; d += 256) out[t * n + d] = from_f<act_t>(to_f(x[d]) * inv * gain[d]);
}

extern "C" const char* sl_slice_rmsnorm(const void* buf, int stride, int col, int n, const float* gain, float eps,
                                        int T, void* out, hipStream_t stream) {
  SL_CHECK(T >= 0 && n > 0 && col >= 0 && col + n <= stride, "slice_rmsnorm: the slice does not fit the rows");
  SL_CHECK(gain != nullptr, "slice_rmsnorm: the gain is required");
  if (T == 0) return nullptr;
  slice_rmsnorm_kernel<<<T, 256, 0, stream>>>((const act_t*)buf, stride, col, n, gain, eps, (act_t*)out);
  return sl_launch_status();
}
