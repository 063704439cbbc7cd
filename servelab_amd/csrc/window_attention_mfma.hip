// The window attention of window_attention.hip on the matrix cores, bfloat16 only, for key widths
// SL_DK (a multiple of 32) and value widths SL_DV (a multiple of 16) fixed at compile time;
// SL_VK = 1: values are the first SL_DV channels of the key rows.  Same call, same meaning.
//
// What is float stays float.  The scores are products of bfloat16 numbers added up in float by
// the matrix instruction (every product is exact in float); scale, cap, distance bias, mask, the
// running maximum and sum and the exponentials are float vector code.  A weight p is not rounded
// to bfloat16 for the second product: it is cut into three bfloat16 terms p = p1 + p2 + p3 (each
// the upper 16 bits of what the terms before left over, 8 bits of significand a term), which
// together are the float exactly, and the weighted sum of the values is three matrix
// instructions, one per term, on float accumulators.
//
// Work layout.  A column is a (token, query head) pair of one sequence and one kv head; a
// wavefront owns 16 columns, a workgroup of four wavefronts 64 consecutive ones, and walks the
// blocks of 32 keys any of them sees.  A block is staged in LDS once for the workgroup: the key
// rows [32][SL_DK], and the values channel-major [SL_DV][32] (copied from the value pages, which
// are channel-major already, or turned in registers, 8 keys x 8 channels a thread, on their way
// from the key rows); the next block is on its way from the pages to registers while a block is
// computed.  Per block and wavefront:
//   S^T[key, column] = K[key, :] . Q[column, :]          mfma 16x16x32, A = K rows, B = Q (registers)
//   O^T[d, column] += V^T[d, key] P^T[key, column]       mfma 16x16x32, A = V^T rows, B = the terms of P
// Row i of score tile m is key 8 (i / 4) + 4 m + i % 4 of the block, so that a lane ends up with
// the weights of 8 consecutive keys of its column: the B operand of the second product as it is.
// A step of single tokens has few columns (the heads of a group): its blocks are cut into shares
// over workgroups, whose wavefronts without a column only help to stage.
#include "window_attention.h"

#if defined(SL_F32)
#error "window_attention_mfma is a bfloat16 kernel; the float32 path uses window_attention.hip"
#endif
#if !defined(SL_DK) || !defined(SL_DV) || !defined(SL_VK)
#error "SL_DK, SL_DV and SL_VK must be defined"
#endif
#if SL_DK % 32 != 0 || SL_DV % 16 != 0 || SL_DK < 32 || SL_DV < 16 || SL_DV > 512 || SL_DK > 1024
#error "SL_DK must be a multiple of 32 up to 1024, SL_DV a multiple of 16 up to 512"
#endif
#if SL_VK && SL_DV > SL_DK
#error "values read from key rows cannot be wider than a key"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int DK = SL_DK, DV = SL_DV;
constexpr bool VK = SL_VK != 0;
constexpr int KK = DK / 32, DD = DV / 16;
constexpr int KROW = DK + 8;          // elements of a staged key row (the pad spreads rows over the banks)
constexpr int VROW = 40;              // elements of a staged channel row: 32 keys and a pad
constexpr float LOG2E = 1.4426950408889634f;

// Maximum / sum over the four lanes n, n + 16, n + 32, n + 48 that share a column, by the row-swap
// instructions of gfx950 (register to register): after a swap of x with itself one result holds
// the lower partner and the other the upper one, in every lane.
__device__ __forceinline__ float column_max4(float x) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float column_sum4(float x) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

constexpr int THREADS = 256, COLS = 64;
constexpr int cdiv(int a, int b) { return (a + b - 1) / b; }
// what a thread stages of a block: chunks of 8 values (16 bytes)
constexpr int KCH = DK / 8;                            // chunks of a key row
constexpr int NKC = VK ? 1 : cdiv(32 * KCH, THREADS);  // key chunks a thread
constexpr int NVC = VK ? 1 : cdiv(DV * 4, THREADS);    // value chunks (a channel's 8 keys) a thread
constexpr int RCH = VK ? (DK - DV) / 8 : 0;            // chunks of a key row behind the values
constexpr int NT = VK ? cdiv((DV / 8) * 4, THREADS) : 1;   // 8 keys x 8 channels tiles a thread (turned on their way into LDS)
constexpr int NR = VK ? (RCH ? cdiv(32 * RCH, THREADS) : 1) : 1;

__global__ __launch_bounds__(THREADS) void window_attention_mfma_kernel(const WindowAttention a) {
  extern __shared__ __attribute__((aligned(16))) __bf16 lds16[];
  __bf16* ks = lds16;                                  // [32][KROW]
  __bf16* vt = ks + 32 * KROW;                         // [DV][VROW]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 15, gq = lane >> 4;
  const int page = a.page, nkv = a.nkv;
  const int seq = blockIdx.z, kvh = blockIdx.y;
  const int g = a.nh / nkv;
  const int q0 = a.cu_q[seq], qlen = a.cu_q[seq + 1] - q0;
  const int ncols = qlen * g;
  const int tile = blockIdx.x / a.nsplit, share = blockIdx.x % a.nsplit;
  const int c0 = tile * COLS;
  if (c0 >= ncols) return;
  const int pos0 = a.positions[q0];
  const int* table = a.tables + (size_t)seq * a.max_pages;

  // the keys any column of the workgroup sees: [0, keep) and [kmin, kmax], as blocks of 32
  const int tok_first = c0 / g;
  const int c_last = c0 + COLS - 1 < ncols - 1 ? c0 + COLS - 1 : ncols - 1;
  const int kmax = pos0 + c_last / g;
  int kmin = 0;
  if (a.window > 0 && pos0 + tok_first - a.window + 1 > 0) kmin = pos0 + tok_first - a.window + 1;
  const int keep = a.keep_first < kmin ? a.keep_first : kmin;
  const int nA = keep > 0 ? (keep - 1) / 32 + 1 : 0;
  int firstB = kmin / 32;
  if (firstB < nA) firstB = nA;
  const int nB = kmax / 32 - firstB + 1 > 0 ? kmax / 32 - firstB + 1 : 0;
  const int nblk = nA + nB;
  const int i0 = (int)((long long)nblk * share / a.nsplit);
  const int i1 = (int)((long long)nblk * (share + 1) / a.nsplit);
  // The blocks are walked from the nearest keys to the farthest (the kept first tokens last): a distance
  // bias makes nearer keys score higher, so the running maximum settles in the first block or two and
  // the sums are rarely rescaled; without a bias the order does not matter.
  auto block_base = [&](int i) {
    const int b = nblk - 1 - i;
    return (b < nA ? b : firstB + (b - nA)) * 32;
  };
  auto loadable = [&](int key) { return key <= kmax && (key >= kmin || key < keep); };

  // this wavefront's columns, and this lane's (a column past the last is computed like the last, never stored)
  const int cw0 = c0 + 16 * wave;
  const bool wave_live = cw0 < ncols;
  const int cw1 = cw0 + 15 < ncols - 1 ? cw0 + 15 : ncols - 1;
  int c = cw0 + n;
  const bool live = c < ncols;
  if (!live) c = ncols - 1;
  const int tok = c / g, head = kvh * g + c % g;
  const int pos_c = pos0 + tok;
  const int lo_c = a.window > 0 && pos_c - a.window + 1 > 0 ? pos_c - a.window + 1 : 0;
  // every column of the wavefront sees all of a block [kb, kb + 31] when kb + 31 <= pos_lo and (kb >= lo_hi
  // or the block lies within the kept first tokens)
  const int pos_lo = pos0 + (wave_live ? cw0 : 0) / g, pos_hi = pos0 + (wave_live ? cw1 : 0) / g;
  const int lo_hi = a.window > 0 && pos_hi - a.window + 1 > 0 ? pos_hi - a.window + 1 : 0;
  const float scale2 = a.scale * LOG2E;
  const bool capped = a.softcap > 0.f;
  const float cap2 = a.softcap * LOG2E, uncap = capped ? a.scale / a.softcap : 0.f;
  const float slope2 = a.slopes != nullptr ? a.slopes[head] * LOG2E : 0.f;
  bf16x8 qf[KK];
  {
    const __bf16* qp = a.q + (size_t)(q0 + tok) * a.q_stride + (size_t)head * DK + 8 * gq;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) qf[kk] = *(const bf16x8*)(qp + 32 * kk);
  }
  f32x4 o[DD];
#pragma unroll
  for (int dd = 0; dd < DD; ++dd) o[dd] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;                        // the maximum in units of log 2
  const __bf16 zero = (__bf16)0.f;
  const bf16x8 zeros = {zero, zero, zero, zero, zero, zero, zero, zero};

  // A block travels pages -> registers -> LDS; the registers are filled for block i + 1 while block i
  // is computed from LDS.
  // The pages of a block (of its keys 0..15 and 16..31) are asked for one block earlier still, so
  // that a block costs one trip to memory and not two in a row; by a vector load (an even lane
  // asks for the first, an odd lane for the second) so that the wait for it is not the wait for LDS.
  const int page_shift = __builtin_ctz(page);
  auto ask_pages = [&](int kbase) {
    const int key = kbase + ((lane & 1) << 4);
    return table[(key <= kmax ? key : kbase) >> page_shift];
  };
  bf16x8 kreg[NKC], vreg[NVC], treg[NT][8], rreg[NR];
  auto fetch = [&](int kbase, int asked) {
    const int pgA = __builtin_amdgcn_readlane(asked, 0), pgB = __builtin_amdgcn_readlane(asked, 1);
    auto key_row = [&](int kl) {                       // start of the cache row of key kbase + kl
      const int pg = kl < 16 ? pgA : pgB;
      return a.kc + (((size_t)pg * nkv + kvh) * page + ((kbase + kl) & (page - 1))) * DK;
    };
    if constexpr (!VK) {
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int idx = tid + THREADS * i, kl = idx / KCH, c8 = idx % KCH;
        kreg[i] = zeros;
        if (idx < 32 * KCH && loadable(kbase + kl)) kreg[i] = *(const bf16x8*)(key_row(kl) + 8 * c8);
      }
#pragma unroll
      for (int i = 0; i < NVC; ++i) {
        const int idx = tid + THREADS * i, d = idx / 4, k8 = idx % 4, key0 = kbase + 8 * k8;
        vreg[i] = zeros;
        if (idx < DV * 4 && key0 <= kmax && (key0 + 7 >= kmin || key0 < keep)) {
          const int pg = k8 < 2 ? pgA : pgB;
          bf16x8 v = *(const bf16x8*)(a.vc + (((size_t)pg * nkv + kvh) * DV + d) * page + (key0 & (page - 1)));
          if (!((key0 + 7 <= kmax && key0 >= kmin) || key0 + 7 < keep)) {
#pragma unroll
            for (int e = 0; e < 8; ++e)                // a slot of the page that holds no visible key may hold anything
              if (!loadable(key0 + e)) v[e] = zero;
          }
          vreg[i] = v;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int idx = tid + THREADS * i, cb = idx / 4, kg = idx % 4;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          treg[i][j] = zeros;
          if (idx < (DV / 8) * 4 && loadable(kbase + 8 * kg + j))
            treg[i][j] = *(const bf16x8*)(key_row(8 * kg + j) + 8 * cb);
        }
      }
      if constexpr (RCH > 0) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const int idx = tid + THREADS * i, kl = idx / RCH, c8 = DV / 8 + idx % RCH;
          rreg[i] = zeros;
          if (idx < 32 * RCH && loadable(kbase + kl)) rreg[i] = *(const bf16x8*)(key_row(kl) + 8 * c8);
        }
      }
    }
  };
  auto store = [&]() {
    if constexpr (!VK) {
#pragma unroll
      for (int i = 0; i < NKC; ++i) {
        const int idx = tid + THREADS * i, kl = idx / KCH, c8 = idx % KCH;
        if (idx < 32 * KCH) *(bf16x8*)(ks + kl * KROW + 8 * c8) = kreg[i];
      }
#pragma unroll
      for (int i = 0; i < NVC; ++i) {
        const int idx = tid + THREADS * i, d = idx / 4, k8 = idx % 4;
        if (idx < DV * 4) *(bf16x8*)(vt + d * VROW + 8 * k8) = vreg[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < NT; ++i) {
        const int idx = tid + THREADS * i, cb = idx / 4, kg = idx % 4;
        if (idx < (DV / 8) * 4) {
#pragma unroll
          for (int j = 0; j < 8; ++j) *(bf16x8*)(ks + (8 * kg + j) * KROW + 8 * cb) = treg[i][j];
#pragma unroll
          for (int e = 0; e < 8; ++e) {                // channel 8 cb + e of the tile's 8 keys
            bf16x8 t;
#pragma unroll
            for (int j = 0; j < 8; ++j) t[j] = treg[i][j][e];
            *(bf16x8*)(vt + (8 * cb + e) * VROW + 8 * kg) = t;
          }
        }
      }
      if constexpr (RCH > 0) {
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const int idx = tid + THREADS * i, kl = idx / RCH, c8 = DV / 8 + idx % RCH;
          if (idx < 32 * RCH) *(bf16x8*)(ks + kl * KROW + 8 * c8) = rreg[i];
        }
      }
    }
  };

  int asked = 0;
  if (i0 < i1) {
    fetch(block_base(i0), ask_pages(block_base(i0)));
    if (i0 + 1 < i1) asked = ask_pages(block_base(i0 + 1));
  }
  for (int i = i0; i < i1; ++i) {
    const int kbase = block_base(i);
    __syncthreads();                                   // the last block's readers are done
    store();
    __syncthreads();
    if (i + 1 < i1) {
      fetch(block_base(i + 1), asked);
      if (i + 2 < i1) asked = ask_pages(block_base(i + 2));
    }
    if (!wave_live) continue;                          // (a wavefront without columns only helps staging)

    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
    const __bf16* kp = ks + (8 * (n / 4) + n % 4) * KROW + 8 * gq;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const bf16x8 k0 = *(const bf16x8*)(kp + 32 * kk);
      const bf16x8 k1 = *(const bf16x8*)(kp + 4 * KROW + 32 * kk);
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k0, qf[kk], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k1, qf[kk], s1, 0, 0, 0);
    }
    // score of key kbase + 8 gq + j: raw * scale - slope * (pos_c - key), in units of log 2
    const float bias0 = -slope2 * (float)(pos_c - kbase - 8 * gq);
    float s[8], top = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float raw = j < 4 ? s0[j] : s1[j - 4];
      s[j] = capped ? fmaf(tanhf(raw * uncap), cap2, fmaf(slope2, (float)j, bias0))
                    : fmaf(raw, scale2, fmaf(slope2, (float)j, bias0));
    }
    const bool whole = kbase + 31 <= pos_lo && (kbase >= lo_hi || kbase + 31 < a.keep_first);
    if (!whole) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = kbase + 8 * gq + j;
        if (!(key <= pos_c && (key >= lo_c || key < a.keep_first))) s[j] = -INFINITY;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) top = fmaxf(top, s[j]);
    const float mn = fmaxf(m, column_max4(top));
    float p[8], psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {                      // exp2(-inf) = 0; mn = -inf only while no key was seen
      p[j] = mn == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(s[j] - mn);
      psum += p[j];
    }
    if (__any(mn > m)) {                               // the maximum of some column moved: rescale
      const float alpha = mn == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(m - mn);
      l *= alpha;
#pragma unroll
      for (int dd = 0; dd < DD; ++dd) o[dd] *= alpha;
      m = mn;
    }
    l += column_sum4(psum);
    // p = p1 + p2 + p3 exactly: each term is the upper 16 bits (a bfloat16) of what the terms before left
    // over, 8 bits of significand a term; two terms of neighbouring keys share a register
    u32x4 w1, w2, w3;
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      unsigned t1[2], t2[2], t3[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float x = p[j + e];
        t1[e] = __float_as_uint(x) & 0xffff0000u;
        const float r1 = x - __uint_as_float(t1[e]);
        t2[e] = __float_as_uint(r1) & 0xffff0000u;
        t3[e] = __float_as_uint(r1 - __uint_as_float(t2[e]));
      }
      w1[j / 2] = __builtin_amdgcn_perm(t1[1], t1[0], 0x07060302u);
      w2[j / 2] = __builtin_amdgcn_perm(t2[1], t2[0], 0x07060302u);
      w3[j / 2] = __builtin_amdgcn_perm(t3[1], t3[0], 0x07060302u);
    }
    const bf16x8 p1 = __builtin_bit_cast(bf16x8, w1), p2 = __builtin_bit_cast(bf16x8, w2),
                 p3 = __builtin_bit_cast(bf16x8, w3);
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) {
      const bf16x8 vf = *(const bf16x8*)(vt + (16 * dd + n) * VROW + 8 * gq);
      f32x4 acc = o[dd];
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p3, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p2, acc, 0, 0, 0);
      o[dd] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, p1, acc, 0, 0, 0);
    }
  }
  if (!live) return;
  // this lane holds channels 16 dd + 4 gq .. + 3 of its column
  const size_t row = (size_t)(q0 + tok) * a.nh + head;
  if (a.nsplit > 1) {
    float* po = a.part_o + (row * a.nsplit + share) * DV + 4 * gq;
#pragma unroll
    for (int dd = 0; dd < DD; ++dd) *(f32x4*)(po + 16 * dd) = o[dd];
    if (gq == 0) {
      a.part_ml[(row * a.nsplit + share) * 2] = m == -INFINITY ? m : m * (1.f / LOG2E);
      a.part_ml[(row * a.nsplit + share) * 2 + 1] = l;
    }
    return;
  }
  // every query sees itself, so m is finite here
  float top = m, extra = 0.f;
  if (a.sinks != nullptr) {
    const float sink2 = a.sinks[head] * LOG2E;
    top = fmaxf(m, sink2);
    extra = __builtin_amdgcn_exp2f(sink2 - top);
  }
  const float w = __builtin_amdgcn_exp2f(m - top);
  float f = w / (l * w + extra);
  if (a.gate != nullptr) f *= sigmoidf_(to_f(a.gate[(size_t)(q0 + tok) * a.gate_stride + head]));
  __bf16* op = a.out + row * DV + 4 * gq;
#pragma unroll
  for (int dd = 0; dd < DD; ++dd) {
    bf16x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = (__bf16)(o[dd][e] * f);
    *(bf16x4*)(op + 16 * dd) = r;
  }
}

static const char* launch_mfma(const WindowAttention& a, dim3 grid, hipStream_t stream) {
  const size_t bytes = sizeof(__bf16) * ((size_t)32 * KROW + (size_t)DV * VROW);
  if (bytes > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)window_attention_mfma_kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return hipGetErrorString(e);
  }
  window_attention_mfma_kernel<<<grid, THREADS, bytes, stream>>>(a);
  return sl_launch_status();
}

extern "C" int sl_window_attention_mfma_lds_bytes() {
  return (int)(sizeof(__bf16) * ((size_t)32 * KROW + (size_t)DV * VROW));
}

// The call of sl_window_attention, for Dk == SL_DK, Dv == SL_DV and (vc == nullptr) == SL_VK.
// q rows, key rows and value rows must be 16-byte aligned.
extern "C" const char* sl_window_attention_mfma(
    const void* q, int q_stride, const void* kc, const void* vc, const int* tables, int max_pages,
    const int* cu_q, const int* positions, int num_seqs, int max_q_len, int num_tokens, int nh,
    int nkv, int Dk, int Dv, int page, float scale, float softcap, int window, int keep_first, const float* slopes,
    const float* sinks, const void* gate, int gate_stride, void* out, int nsplit, float* part_o,
    float* part_ml, hipStream_t stream) {
  SL_CHECK(Dk == DK && Dv == DV && (vc == nullptr) == VK, "window attention (matrix cores): built for other widths");
  SL_CHECK(num_seqs >= 0 && max_q_len >= 1 && nh > 0 && nkv > 0 && nh % nkv == 0,
           "window attention: heads must be a positive multiple of kv heads");
  SL_CHECK(page == 16 || page == 32 || page == 64, "window attention: page size must be 16, 32 or 64");
  SL_CHECK(nkv <= 65535 && num_seqs <= 65535, "window attention: grid too large");
  SL_CHECK(window >= 0 && keep_first >= 0 && softcap >= 0.f, "window attention: window, keep_first and the cap must be >= 0");
  SL_CHECK(nsplit >= 1 && nsplit <= 64, "window attention: 1..64 shares of the keys");
  SL_CHECK(nsplit == 1 || (part_o != nullptr && part_ml != nullptr),
           "window attention: shares of the keys need the partial buffers");
  SL_CHECK(gate == nullptr || gate_stride >= nh, "window attention: gate rows are shorter than the heads");
  SL_CHECK((uintptr_t)q % 16 == 0 && q_stride % 8 == 0 && (uintptr_t)kc % 16 == 0 && (uintptr_t)vc % 16 == 0 &&
           (uintptr_t)out % 8 == 0 && (uintptr_t)part_o % 16 == 0,
           "window attention (matrix cores): operands must be 16-byte aligned");
  if (num_seqs == 0 || num_tokens == 0) return nullptr;
  const WindowAttention a{(const act_t*)q, q_stride, (const act_t*)kc, (const act_t*)vc, tables, max_pages,
                          cu_q, positions, nh, nkv, Dk, Dv, page, scale, softcap, window, keep_first, slopes, sinks,
                          (const act_t*)gate, gate_stride, (act_t*)out, nsplit, part_o, part_ml};
  const long long cols = (long long)max_q_len * (nh / nkv);
  const long long tiles = (cols + COLS - 1) / COLS;
  SL_CHECK(tiles * nsplit <= 1 << 30, "window attention: too many column tiles");
  const dim3 grid((unsigned)(tiles * nsplit), nkv, num_seqs);
  const char* e = launch_mfma(a, grid, stream);
  if (e || nsplit == 1) return e;
  window_attention_combine_kernel<<<dim3(num_tokens, nh, (Dv + 63) / 64), 64, 0, stream>>>(
      part_o, part_ml, nsplit, nh, Dv, sinks, (const act_t*)gate, gate_stride, (act_t*)out);
  return sl_launch_status();
}
