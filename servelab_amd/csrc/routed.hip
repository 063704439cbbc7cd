// Routed experts: every token goes through the `top` experts with the largest router logits,
// weighted by the softmax over those logits only; or (shares over all experts) with the largest
// softmax shares plus a correction per expert, weighted by their shares, divided by their sum
// and multiplied by a constant.  The last experts may be ones without matrices that hand their
// input through.
//
//   route       per token the chosen experts and their shares (float), one wavefront a token
//   group       the step's (token, choice) pairs sorted by expert, on the device: where each
//               expert's rows start, the list of row tiles (expert, first row, rows) that the
//               grouped products walk, and each pair's place in the sorted order
//   grouped     y[row] = W[expert of row] x[row]: one launch over all experts, a workgroup per
//               (row tile, column tile); the gated form computes act(gate) * up of an expert's
//               stacked [gate; up] matrix, the activated form act(W x) of a single one
//   combine     out[token] = g base[token] + sum over its choices of share * y[place of the pair],
//               g = 1 or the sigmoid of one number per token
//
// No launch depends on the routing: the grids are sized for the worst case (pairs / tile rows
// + experts tiles) and workgroups beyond the tiles in use leave at once, so a step is a fixed
// list of launches that a captured graph can replay.
#include "common.h"

#define RT_ROWS 16           // rows of a tile of the plain grouped product; a row tile holds 16, 64 or 128 rows

// ------------------------------------------------------------------ route
// One wavefront per token.  Largest first; among equal logits the lower index wins.
// over_all: the numbers compared are softmax(z)[e] + correction[e] over all E, and a chosen
// expert's share is softmax(z)[e] / (sum over the chosen + 1e-20) * scale.
__global__ __launch_bounds__(64) void route_kernel(const float* __restrict__ logits, int stride, int E, int top,
                                                   int* __restrict__ chosen, float* __restrict__ shares,
                                                   int over_all, const float* __restrict__ correction,
                                                   float scale) {
  const size_t t = blockIdx.x;
  const int lane = threadIdx.x;
  const float* z = logits + t * stride;
  float zmax = 0.f, inv_sum = 1.f;
  if (over_all) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
    zmax = wave_max(mx);
    float sm = 0.f;
    for (int e = lane; e < E; e += 64) sm += expf(z[e] - zmax);
    inv_sum = 1.f / wave_sum(sm);
  }
  unsigned long long taken = 0ull;             // bit u: element lane + 64 u is chosen already (E <= 4096)
  float mine = 0.f;                            // lane k keeps the k-th largest logit
  int mine_e = 0;
  auto number = [&](int e) -> float {          // what the experts are compared by
    const float v = z[e];
    return over_all ? expf(v - zmax) * inv_sum + (correction != nullptr ? correction[e] : 0.f) : v;
  };
  float kept[4];                               // a lane's first four numbers stay in registers (E <= 256: all)
#pragma unroll
  for (int u = 0; u < 4; ++u) kept[u] = lane + 64 * u < E ? number(lane + 64 * u) : -INFINITY;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int at = 0x7fffffff;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = lane + 64 * u;
      if (e < E && !((taken >> u) & 1ull) && (kept[u] > best || (kept[u] == best && e < at))) {
        best = kept[u];
        at = e;
      }
    }
    for (int u = 4, e = lane + 256; e < E; ++u, e += 64) {
      const float v = number(e);
      if (!((taken >> u) & 1ull) && (v > best || (v == best && e < at))) {
        best = v;
        at = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, SL_WAVE);
      const int oa = __shfl_xor(at, o, SL_WAVE);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (at % 64 == lane) taken |= 1ull << (at / 64);
    if (lane == k) {
      mine = best;
      mine_e = at;
    }
  }
  if (over_all) {
    const float w = lane < top ? expf(z[mine_e] - zmax) * inv_sum : 0.f;
    const float sum = wave_sum(w);
    if (lane < top) {
      chosen[t * top + lane] = mine_e;
      shares[t * top + lane] = w / (sum + 1e-20f) * scale;
    }
    return;
  }
  const float top1 = __shfl(mine, 0, SL_WAVE);
  const float w = lane < top ? expf(mine - top1) : 0.f;
  const float sum = wave_sum(w);
  if (lane < top) {
    chosen[t * top + lane] = mine_e;
    shares[t * top + lane] = w / sum;
  }
}

// ------------------------------------------------------------------ group
// One workgroup sorts the n = tokens * top pairs by expert (counting sort in LDS).
//   order[place] = pair (token * top + choice);  place_of[pair] = place
//   tiles[i] = {expert, first row, rows} for i < tiles in use; rows 0 beyond
// Experts from E_real on have no matrices: their pairs get places but no tiles.
__global__ __launch_bounds__(1024) void group_kernel(const int* __restrict__ chosen, int n, int E, int E_real, int max_tiles,
                                                     int tile_rows, int* __restrict__ order,
                                                     int* __restrict__ place_of, int* __restrict__ tiles) {
  extern __shared__ int sh[];
  int* count = sh;               // [E]
  int* start = sh + E;           // [E] first row of the expert
  int* tile0 = sh + 2 * E;       // [E] first tile of the expert
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += blockDim.x) count[e] = 0;
  for (int i = tid; i < max_tiles; i += blockDim.x) {
    tiles[3 * i] = 0;
    tiles[3 * i + 1] = 0;
    tiles[3 * i + 2] = 0;
  }
  __syncthreads();
  for (int i = tid; i < n; i += blockDim.x) atomicAdd(&count[chosen[i]], 1);
  __syncthreads();
  if (tid == 0) {
    int rows = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = rows;
      tile0[e] = nt;
      rows += count[e];
      if (e < E_real) nt += (count[e] + tile_rows - 1) / tile_rows;
    }
  }
  __syncthreads();
  for (int e = tid; e < E_real; e += blockDim.x) {
    const int c = count[e];
    for (int i = 0; i * tile_rows < c; ++i) {
      int* tl = tiles + 3 * (tile0[e] + i);
      tl[0] = e;
      tl[1] = start[e] + i * tile_rows;
      tl[2] = min(tile_rows, c - i * tile_rows);
    }
  }
  __syncthreads();
  for (int e = tid; e < E; e += blockDim.x) count[e] = start[e];      // now the next free row
  __syncthreads();
  for (int i = tid; i < n; i += blockDim.x) {
    const int place = atomicAdd(&count[chosen[i]], 1);
    order[place] = i;
    place_of[i] = place;
  }
}

extern "C" const char* sl_route_tokens(const float* logits, int stride, int T, int E, int top, int* chosen,
                                       float* shares, int* order, int* place_of, int* tiles, int max_tiles,
                                       int tile_rows, int over_all, const float* correction, float scale,
                                       int E_real, hipStream_t stream) {
  SL_CHECK(T >= 0 && E >= 1 && E <= 4096 && top >= 1 && top <= 64 && top <= E && E <= stride,
           "route_tokens: at most 4096 experts within the rows, at most 64 choices");
  SL_CHECK(E_real >= 0 && E_real <= E && (over_all || correction == nullptr),
           "route_tokens: the experts with matrices are the first of all; a correction needs shares over all");
  SL_CHECK(tile_rows == 16 || tile_rows == 64 || tile_rows == 128, "route_tokens: row tiles hold 16, 64 or 128 rows");
  SL_CHECK(max_tiles >= ((long long)T * top + tile_rows - 1) / tile_rows + E, "route_tokens: too few tile entries");
  if (T == 0) return nullptr;
  route_kernel<<<T, 64, 0, stream>>>(logits, stride, E, top, chosen, shares, over_all, correction, scale);
  group_kernel<<<1, 1024, 3 * E * sizeof(int), stream>>>(chosen, T * top, E, E_real, max_tiles, tile_rows, order,
                                                         place_of, tiles);
  return sl_launch_status();
}

// ------------------------------------------------------------------ grouped products
struct Grouped {
  const act_t* x;            // row r reads x + src(r) * K, src(r) = order[r] / top when order is given, else r
  const int* order;
  int top;
  const act_t* w;            // [experts][N_w][K]; gated: N_w = 2 N, gate rows before up rows
  int w_tiled;               // an expert's matrix lies as [N_w / 16][K / 32][64 lanes][8], lane = 16 (k / 8 % 4) + n % 16:
                             // the first operand of mfma 16x16x32 as it sits in registers, 1 KB a wavefront's load
  const int* tiles;          // [max_tiles][3]
  int sub;                   // row tiles hold 16 * sub rows
  int N, K;
  act_t* out_act;            // gated and activated: [rows][N]
  float* out_f32;            // plain: [rows][N]
  int act;                   // the activation (common.h); 0 with out_f32
  float limit;               // the clamped gate's bound
  int max_tiles, col_blocks; // the matrix-core kernels' launch: max_tiles x col_blocks workgroups in a row
};

// Which (row tile, column block) a workgroup of a one-dimensional launch takes.  Workgroups go to the
// chip's eight dies in turn (number % 8), and each die has an L2 of its own: a die gets a contiguous
// run of the list ordered by column block, then row tile, so the row tiles of one expert, which read
// the same columns of the same matrices, run on one die at about the same time and the matrices
// come from memory once.
__device__ __forceinline__ bool grouped_place(const Grouped& a, int& tile, int& cb) {
  const int total = a.max_tiles * a.col_blocks, run = (total + 7) / 8;
  const int m = (blockIdx.x & 7) * run + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= run || m >= total) return false;
  cb = m / a.max_tiles;
  tile = m - cb * a.max_tiles;
  return true;
}

// 256 threads: thread (row = tid / 16, lane16 = tid % 16) owns columns lane16 + 16 u, u < 4, of a
// 16 x 64 tile.  x and W go through LDS in chunks of 32 values of k; sums are float.
template <bool GATED>
__global__ __launch_bounds__(256) void grouped_product_kernel(const Grouped a) {   // (not GATED: plain or activated)
  const int* tl = a.tiles + 3 * (blockIdx.x / a.sub);
  const int part = blockIdx.x % a.sub;                  // which 16 rows of the row tile
  const int rows = min(RT_ROWS, tl[2] - RT_ROWS * part);
  if (rows <= 0) return;
  const int e = tl[0], row0 = tl[1] + RT_ROWS * part;
  const int n0 = blockIdx.y * 64;
  __shared__ float xs[RT_ROWS][33];
  __shared__ float ws[GATED ? 128 : 64][33];
  const int tid = threadIdx.x, r = tid / 16, l = tid % 16;
  const size_t n_w = GATED ? 2 * (size_t)a.N : (size_t)a.N;
  const act_t* we = a.w + (size_t)e * n_w * a.K;
  float acc[4] = {0.f, 0.f, 0.f, 0.f}, acc2[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < a.K; k0 += 32) {
    __syncthreads();
    for (int i = tid; i < RT_ROWS * 32; i += 256) {
      const int rr = i / 32, kk = i % 32;
      float v = 0.f;
      if (rr < rows && k0 + kk < a.K) {
        const size_t src = a.order != nullptr ? (size_t)(a.order[row0 + rr] / a.top) : (size_t)(row0 + rr);
        v = to_f(a.x[src * a.K + k0 + kk]);
      }
      xs[rr][kk] = v;
    }
    for (int i = tid; i < (GATED ? 128 : 64) * 32; i += 256) {
      const int c = i / 32, kk = i % 32;
      const int n = n0 + (c % 64);
      float v = 0.f;
      if (n < a.N && k0 + kk < a.K) v = to_f(we[((size_t)(c / 64) * a.N + n) * a.K + k0 + kk]);
      ws[c][kk] = v;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < 32; ++kk) {
      const float xv = xs[r][kk];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        acc[u] += xv * ws[l + 16 * u][kk];
        if (GATED) acc2[u] += xv * ws[64 + l + 16 * u][kk];
      }
    }
  }
  if (r >= rows) return;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int n = n0 + l + 16 * u;
    if (n >= a.N) continue;
    const size_t at = (size_t)(row0 + r) * a.N + n;
    if (GATED) a.out_act[at] = from_f<act_t>(sl_gated(acc[u], acc2[u], a.act, a.limit));
    else if (a.act) a.out_act[at] = from_f<act_t>(sl_act(acc[u], a.act));
    else a.out_f32[at] = acc[u];
  }
}

#if !defined(SL_F32)
typedef __bf16 rt_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 rt_bf16x4 __attribute__((ext_vector_type(4)));
typedef float rt_f32x4 __attribute__((ext_vector_type(4)));

// The same on the matrix cores (bfloat16, K in steps of 32, N in steps of 16): a wavefront owns
// NT x 16 rows of a row tile by NU x 16 columns and reads its operands straight from
// memory, eight values a lane: rows of W are the first operand of mfma 16x16x32, rows of x the
// second; the gated form keeps gate and up sums of the same columns.  Rows past the tile's last are
// computed like the last and never stored.
template <int NT, int NU, bool GATED, int WR, int WC>
__global__ __launch_bounds__(64 * WR * WC) void grouped_product_mfma_kernel(const Grouped a) {
  // WR x WC wavefronts a workgroup: WR along the rows of the row tile, WC along the columns; those
  // that read the same rows of x or of W find them in the CU's cache after the first has asked
  int tile, cb;
  if (!grouped_place(a, tile, cb)) return;
  const int* tl = a.tiles + 3 * tile;
  const int wave = threadIdx.x / 64, wr = wave % WR, wc = wave / WR;
  const int rows = min(16 * NT, tl[2] - 16 * NT * wr);
  const int n0 = (cb * WC + wc) * 16 * NU;
  if (rows <= 0 || n0 >= a.N) return;
  const int e = tl[0], row0 = tl[1] + 16 * NT * wr;
  const int lane = threadIdx.x & 63, i = lane & 15, gq = lane >> 4;
  const size_t n_w = GATED ? 2 * (size_t)a.N : (size_t)a.N;
  const __bf16* we = a.w + (size_t)e * n_w * a.K;
  const __bf16* xp[NT];
#pragma unroll
  for (int v = 0; v < NT; ++v) {
    const int rr = row0 + min(16 * v + i, rows - 1);
    const size_t src = a.order != nullptr ? (size_t)(a.order[rr] / a.top) : (size_t)rr;
    xp[v] = a.x + src * a.K + 8 * gq;
  }
  const __bf16* wp[NU];
  const int wstep = a.w_tiled ? 512 : 32;               // elements from one k-step to the next
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    if (a.w_tiled) wp[u] = we + (size_t)(min(n0 + 16 * u, a.N - 16) / 16) * (a.K / 32) * 512 + lane * 8;
    else wp[u] = we + (size_t)min(n0 + 16 * u + i, a.N - 1) * a.K + 8 * gq;
  }
  const size_t up = (size_t)a.N * a.K;                  // from a gate row to its up row (N in steps of 16)
  rt_f32x4 acc[NT][NU], acc2[NT][GATED ? NU : 1];
#pragma unroll
  for (int v = 0; v < NT; ++v)
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      acc[v][u] = rt_f32x4{0.f, 0.f, 0.f, 0.f};
      if (GATED) acc2[v][u] = rt_f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll 4
  for (int k = 0; k < a.K; k += 32) {
    rt_bf16x8 b[NT], w1[NU], w2[GATED ? NU : 1];
    const size_t kw = (size_t)(k / 32) * wstep;
#pragma unroll
    for (int v = 0; v < NT; ++v) b[v] = *(const rt_bf16x8*)(xp[v] + k);
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      w1[u] = *(const rt_bf16x8*)(wp[u] + kw);
      if (GATED) w2[u] = *(const rt_bf16x8*)(wp[u] + up + kw);
    }
#pragma unroll
    for (int v = 0; v < NT; ++v)
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        acc[v][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u], b[v], acc[v][u], 0, 0, 0);
        if (GATED) acc2[v][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w2[u], b[v], acc2[v][u], 0, 0, 0);
      }
  }
  // this lane holds columns n0 + 16 u + 4 gq .. + 3 of rows 16 v + i
#pragma unroll
  for (int v = 0; v < NT; ++v) {
    if (16 * v + i >= rows) continue;
    const size_t at = (size_t)(row0 + 16 * v + i) * a.N + n0 + 4 * gq;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      if (n0 + 16 * u >= a.N) continue;
      if (GATED) {
        rt_bf16x4 r;
#pragma unroll
        for (int c = 0; c < 4; ++c) r[c] = (__bf16)sl_gated(acc[v][u][c], acc2[v][u][c], a.act, a.limit);
        *(rt_bf16x4*)(a.out_act + at + 16 * u) = r;
      } else if (a.act) {
        rt_bf16x4 r;
#pragma unroll
        for (int c = 0; c < 4; ++c) r[c] = (__bf16)sl_act(acc[v][u][c], a.act);
        *(rt_bf16x4*)(a.out_act + at + 16 * u) = r;
      } else {
        *(rt_f32x4*)(a.out_f32 + at + 16 * u) = acc[v][u];
      }
    }
  }
}


// Row tiles of 128 rows with the rows of x staged in LDS: a workgroup of four wavefronts takes a row
// tile by 64 NU columns; every wavefront owns all 128 rows by 16 NU columns (of the gate and of the
// up matrix in the gated form).  The tile's rows of x come 64 values of k at a time into one of two
// halves of LDS (a thread brings four 16-byte pieces, asked for one step ahead); a row's eight pieces
// are stored at piece ^ (row / 2 % 8), so that the 16 lanes of a fragment read, and the 16 of a
// write, take every bank once.  W comes straight from memory in the tiled layout, a k-step ahead: no
// two wavefronts of the workgroup read the same piece of it, and the CU's cache delivers a third of
// what the unstaged kernel asks of it.  Two workgroups a CU: one computes while the other waits.
template <int NU, bool GATED>
__global__ __launch_bounds__(256, 2) void grouped_product_staged_kernel(const Grouped a) {
  constexpr int NT = 8, MATS = GATED ? 2 : 1;
  __shared__ __attribute__((aligned(16))) __bf16 stage[2][128 * 64];
  int tile, cb;
  if (!grouped_place(a, tile, cb)) return;
  const int* tl = a.tiles + 3 * tile;
  const int rows = min(128, tl[2]);
  if (rows <= 0) return;                                // (the whole workgroup: no barrier is left waiting)
  const int e = tl[0], row0 = tl[1];
  const int wave = threadIdx.x / 64, lane = threadIdx.x & 63, i = lane & 15, gq = lane >> 4;
  const int n0 = (cb * 4 + wave) * 16 * NU;
  const size_t n_w = GATED ? 2 * (size_t)a.N : (size_t)a.N;
  const __bf16* we = a.w + (size_t)e * n_w * a.K;
  const size_t up = (size_t)a.N * a.K;
  const __bf16* wp[NU];
#pragma unroll
  for (int u = 0; u < NU; ++u)
    wp[u] = we + (size_t)(min(n0 + 16 * u, a.N - 16) / 16) * (a.K / 32) * 512 + lane * 8;
  // what this thread brings: piece threadIdx % 8 of rows threadIdx / 8 + 32 j
  const int piece = threadIdx.x & 7, rbase = threadIdx.x >> 3;
  const __bf16* xsrc[4];
  int xat[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = rbase + 32 * j, rr = row0 + min(r, rows - 1);
    const size_t src = a.order != nullptr ? (size_t)(a.order[rr] / a.top) : (size_t)rr;
    xsrc[j] = a.x + src * a.K + 8 * piece;
    xat[j] = r * 64 + 8 * (piece ^ ((r >> 1) & 7));
  }
  const int fsw = (i >> 1) & 7;                         // (16 v + i) / 2 % 8
  rt_f32x4 acc[NT][NU * MATS];
#pragma unroll
  for (int v = 0; v < NT; ++v)
#pragma unroll
    for (int u = 0; u < NU * MATS; ++u) acc[v][u] = rt_f32x4{0.f, 0.f, 0.f, 0.f};
  rt_bf16x8 xr[4], wcur[NU * MATS], wnext[NU * MATS];
#pragma unroll
  for (int j = 0; j < 4; ++j) xr[j] = *(const rt_bf16x8*)(xsrc[j]);
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    wcur[u] = *(const rt_bf16x8*)(wp[u]);
    if (GATED) wcur[NU + u] = *(const rt_bf16x8*)(wp[u] + up);
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) *(rt_bf16x8*)(&stage[0][xat[j]]) = xr[j];
  __syncthreads();
  const int steps = a.K / 64;
  for (int s = 0; s < steps; ++s) {
    if (s + 1 < steps) {
#pragma unroll
      for (int j = 0; j < 4; ++j) xr[j] = *(const rt_bf16x8*)(xsrc[j] + 64 * (s + 1));
    }
    const __bf16* buf = stage[s & 1] + i * 64;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kstep = 2 * s + h;
      if (kstep + 1 < 2 * steps) {
        const size_t kw = (size_t)(kstep + 1) * 512;
#pragma unroll
        for (int u = 0; u < NU; ++u) {
          wnext[u] = *(const rt_bf16x8*)(wp[u] + kw);
          if (GATED) wnext[NU + u] = *(const rt_bf16x8*)(wp[u] + up + kw);
        }
      }
      const int fo = 8 * ((4 * h + gq) ^ fsw);
#pragma unroll
      for (int v = 0; v < NT; ++v) {
        const rt_bf16x8 b = *(const rt_bf16x8*)(buf + v * 16 * 64 + fo);
#pragma unroll
        for (int u = 0; u < NU * MATS; ++u)
          acc[v][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wcur[u], b, acc[v][u], 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < NU * MATS; ++u) wcur[u] = wnext[u];
    }
    if (s + 1 < steps) {
#pragma unroll
      for (int j = 0; j < 4; ++j) *(rt_bf16x8*)(&stage[(s + 1) & 1][xat[j]]) = xr[j];
    }
    __syncthreads();
  }
  // this lane holds columns n0 + 16 u + 4 gq .. + 3 of rows 16 v + i
#pragma unroll
  for (int v = 0; v < NT; ++v) {
    if (16 * v + i >= rows) continue;
    const size_t at = (size_t)(row0 + 16 * v + i) * a.N + n0 + 4 * gq;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      if (n0 + 16 * u >= a.N) continue;
      if (GATED) {
        rt_bf16x4 r;
#pragma unroll
        for (int c = 0; c < 4; ++c) r[c] = (__bf16)sl_gated(acc[v][u][c], acc[v][NU + u][c], a.act, a.limit);
        *(rt_bf16x4*)(a.out_act + at + 16 * u) = r;
      } else if (a.act) {
        rt_bf16x4 r;
#pragma unroll
        for (int c = 0; c < 4; ++c) r[c] = (__bf16)sl_act(acc[v][u][c], a.act);
        *(rt_bf16x4*)(a.out_act + at + 16 * u) = r;
      } else {
        *(rt_f32x4*)(a.out_f32 + at + 16 * u) = acc[v][u];
      }
    }
  }
}
#endif

extern "C" const char* sl_grouped_product(const void* x, const int* order, int top, const void* w, const int* tiles,
                                          int w_tiled, int max_tiles, int tile_rows, int N, int K, int gated,
                                          int act, float limit, void* out, hipStream_t stream) {
  // gated: act(gate) * up into the activation type; else act != 0: act(W x) into the activation type;
  // else plain float sums
  SL_CHECK(max_tiles >= 0 && N > 0 && K > 0 && top >= 1, "grouped_product: sizes must be positive");
  SL_CHECK(act >= 0 && act <= SL_ACT_CLAMPED_SWISH && (!gated || act) && (gated || act != SL_ACT_CLAMPED_SWISH),
           "grouped_product: unknown activation, a gate without one, or the clamped form without a gate");
  SL_CHECK(tile_rows == 16 || tile_rows == 64 || tile_rows == 128, "grouped_product: row tiles hold 16, 64 or 128 rows");
  if (max_tiles == 0) return nullptr;
  Grouped a{(const act_t*)x, order, top, (const act_t*)w, w_tiled, tiles, tile_rows / RT_ROWS, N, K,
            act ? (act_t*)out : nullptr, act ? nullptr : (float*)out, act, limit, max_tiles, 1};
#if !defined(SL_F32)
  if (K % 32 == 0 && N % 16 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)out % 16 == 0) {
    // (a one-dimensional launch of max_tiles x col_blocks workgroups, rounded up to the eight dies)
    auto blocks = [&](int cols) {
      a.col_blocks = (N + cols - 1) / cols;
      return dim3(8 * (unsigned)((max_tiles * a.col_blocks + 7) / 8));
    };
    if (tile_rows == 128 && w_tiled && K % 64 == 0) {   // the tile's rows of x staged in LDS
      if (gated) grouped_product_staged_kernel<2, true><<<blocks(128), 256, 0, stream>>>(a);
      else grouped_product_staged_kernel<4, false><<<blocks(256), 256, 0, stream>>>(a);
    } else if (tile_rows == 128) {                      // two wavefronts along the rows, two along the columns
      if (gated) grouped_product_mfma_kernel<4, 4, true, 2, 2><<<blocks(128), 256, 0, stream>>>(a);
      else grouped_product_mfma_kernel<4, 4, false, 2, 2><<<blocks(128), 256, 0, stream>>>(a);
    } else if (tile_rows == 64) {
      if (gated) grouped_product_mfma_kernel<4, 4, true, 1, 4><<<blocks(256), 256, 0, stream>>>(a);
      else grouped_product_mfma_kernel<4, 4, false, 1, 4><<<blocks(256), 256, 0, stream>>>(a);
    } else {
      if (gated) grouped_product_mfma_kernel<1, 4, true, 1, 1><<<blocks(64), 64, 0, stream>>>(a);
      else grouped_product_mfma_kernel<1, 4, false, 1, 1><<<blocks(64), 64, 0, stream>>>(a);
    }
    return sl_launch_status();
  }
#endif
  SL_CHECK(!w_tiled, "grouped_product: tiled matrices need K in steps of 32, N in steps of 16 and aligned operands");
  const dim3 grid(max_tiles * (tile_rows / RT_ROWS), (N + 63) / 64);
  if (gated) grouped_product_kernel<true><<<grid, 256, 0, stream>>>(a);
  else grouped_product_kernel<false><<<grid, 256, 0, stream>>>(a);
  return sl_launch_status();
}

// ------------------------------------------------------------------ combine
// out[t] = g[t] base[t] + sum_k shares[t][k] * y[place_of[t top + k]], float sums, choices in their order;
// g[t] = sigmoid(base_gate[t * gate_stride]) when base_gate is given, else 1.  A choice from
// E_real on (chosen given) is an expert that hands its input through: it adds share * x[t].
__global__ __launch_bounds__(256) void routed_combine_kernel(const float* __restrict__ y,
                                                             const int* __restrict__ place_of,
                                                             const float* __restrict__ shares, int top,
                                                             const act_t* __restrict__ base,
                                                             const float* __restrict__ base_gate, int gate_stride,
                                                             int H, act_t* __restrict__ out,
                                                             const int* __restrict__ chosen, int E_real,
                                                             const act_t* __restrict__ x) {
  __shared__ int place[64];
  __shared__ float share[64];
  const size_t t = blockIdx.x;
  if (threadIdx.x < top) {
    const bool through = chosen != nullptr && chosen[t * top + threadIdx.x] >= E_real;
    place[threadIdx.x] = through ? -1 : place_of[t * top + threadIdx.x];
    share[threadIdx.x] = shares[t * top + threadIdx.x];
  }
  __syncthreads();
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= H) return;
  float v = base != nullptr ? to_f(base[t * H + c]) : 0.f;
  if (base_gate != nullptr) v *= 1.f / (1.f + expf(-base_gate[t * gate_stride]));
  for (int k = 0; k < top; ++k)
    v += share[k] * (place[k] < 0 ? to_f(x[t * H + c]) : y[(size_t)place[k] * H + c]);
  out[t * H + c] = from_f<act_t>(v);
}

extern "C" const char* sl_routed_combine(const float* y, const int* place_of, const float* shares, int T, int top,
                                         const void* base, const float* base_gate, int gate_stride, int H,
                                         void* out, const int* chosen, int E_real, const void* x,
                                         hipStream_t stream) {
  SL_CHECK(T >= 0 && top >= 1 && top <= 64 && H > 0, "routed_combine: sizes must be positive, at most 64 choices");
  SL_CHECK(chosen == nullptr || x != nullptr, "routed_combine: experts that hand their input through need the input");
  if (T == 0) return nullptr;
  routed_combine_kernel<<<dim3(T, (H + 255) / 256), 256, 0, stream>>>(y, place_of, shares, top, (const act_t*)base,
                                                                    base_gate, gate_stride, H, (act_t*)out,
                                                                    chosen, E_real, (const act_t*)x);
  return sl_launch_status();
}
