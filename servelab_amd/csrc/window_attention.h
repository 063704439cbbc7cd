// What the two window attention sources share (the float kernel for every size and both
// activation types, and the matrix-core kernel for bfloat16): the parameters of a call, and
// the kernel that merges the shares of the keys.
#pragma once
#include "common.h"

struct WindowAttention {
  const act_t* q;            // head h of token t at q + t * q_stride + h * Dk
  int q_stride;
  const act_t* kc;           // [pages][nkv][page][Dk]
  const act_t* vc;           // [pages][nkv][Dv][page], or nullptr: values are key channels [0, Dv)
  const int* tables;         // [sequences][max_pages]
  int max_pages;
  const int* cu_q;           // [sequences + 1]
  const int* positions;      // [tokens]
  int nh, nkv, Dk, Dv, page;
  float scale;
  float softcap;             // c > 0: the scaled score becomes c tanh(score / c); 0: left as it is
  int window;                // 0: every earlier key
  int keep_first;
  const float* slopes;       // [nh] or nullptr
  const float* sinks;        // [nh] or nullptr
  const act_t* gate;         // gate of (t, h) at gate[t * gate_stride + h], or nullptr
  int gate_stride;
  act_t* out;                // [tokens][nh][Dv]
  int nsplit;
  float* part_o;             // [tokens][nh][nsplit][Dv]
  float* part_ml;            // [tokens][nh][nsplit][2]
};

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }

// Merges the shares of a (token, head): out = sum_j w_j o_j / (sum_j w_j l_j + sink's term),
// w_j = exp(m_j - top); a share without keys has m = -inf and drops out.  One
// wavefront per (token, head, 64 channels); shares are added in their order.
__global__ __launch_bounds__(64) void window_attention_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, int nsplit, int nh, int Dv,
    const float* __restrict__ sinks, const act_t* __restrict__ gate, int gate_stride,
    act_t* __restrict__ out) {
  __shared__ float ws[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t base = ((size_t)t * nh + h) * nsplit;
  // lane j holds share j (at most 64 shares)
  float mj = -INFINITY, lj = 0.f;
  if (lane < nsplit) {
    mj = part_ml[(base + lane) * 2];
    lj = part_ml[(base + lane) * 2 + 1];
  }
  const float sink = sinks != nullptr ? sinks[h] : -INFINITY;
  const float top = fmaxf(wave_max(mj), sink);
  const float wj = mj == -INFINITY ? 0.f : expf(mj - top);
  const float denom = wave_sum(wj * lj) + (sinks != nullptr ? expf(sink - top) : 0.f);
  ws[lane] = wj;
  __syncthreads();
  float f = 1.f / denom;
  if (gate != nullptr) f *= sigmoidf_(to_f(gate[(size_t)t * gate_stride + h]));
  act_t* o = out + ((size_t)t * nh + h) * Dv;
  const int d = blockIdx.z * 64 + lane;
  if (d < Dv) {
    float s = 0.f;
    for (int j = 0; j < nsplit; j += 8) {              // eight shares asked for together; added in their order
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = j + u < nsplit ? part_o[(base + j + u) * Dv + d] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) s += (j + u < nsplit ? ws[j + u] : 0.f) * v[u];
    }
    o[d] = from_f<act_t>(s * f);
  }
}
