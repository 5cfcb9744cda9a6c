// Matrix-core form of the windowed pooled attention for bf16 activations and caches.
//
// One workgroup = one tile of 16 consecutive new tokens of one sequence, one kv head, up to four of its
// query heads (one per wave). Keys are walked in tiles of 64 entries, first the pooled blocks that any
// query of the tile may see, then the tokens from the first window start to the last query; what a
// query does not see (outside its window, a block not yet wholly before it, the future) is masked.
//
// Everything is computed transposed so that no operand changes layout between the two products:
//   S^T = K Q^T   v_mfma_f32_16x16x16_bf16, A = 16 keys x 16 of D read straight from the cache rows,
//                 B = the wave's Q fragments (registers, loaded once); a lane ends up with 4 keys of ONE query,
//                 so the softmax statistics of a query live in 4 lanes (two shuffles) and
//   O^T += V^T P^T  takes the probabilities as its B operand exactly as they lie (keys x queries), with
//                 A = V^T read from the 64-entry V tile that the four waves stage in LDS together.
// The sink is the initial state of the running softmax: maximum 0, sum 1.
#include "mix_common.h"

namespace lvmix {

typedef __attribute__((ext_vector_type(4))) short bf16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

struct WindowMfmaParams {
  const uint16_t *q, *k_cache, *v_cache, *kp, *vp, *gate;
  int64_t ld_gate;
  uint16_t* out;
  const int32_t *cu_q, *ctx_lens, *block_tables;
  int bt_stride, H, G, D, Dv, page, window, P, PP, ngroups;
  float scale, sink;
};

constexpr int kTileQ = 16;
constexpr int kTileK = 64;
constexpr int kMaxKK = 16;     // D <= 256
constexpr int kMaxDvb = 16;    // Dv <= 256

__device__ __forceinline__ short bf16_bits(float x) {
  __bf16 b = static_cast<__bf16>(x);
  return __builtin_bit_cast(short, b);
}

__global__ __launch_bounds__(256) void window_pool_mfma_kernel(WindowMfmaParams p) {
  extern __shared__ uint16_t vs[];                      // [kTileK][Dv + 4]
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int ln = lane & 15, lg = lane >> 4;
  const int b = blockIdx.z;
  const int g = blockIdx.y / p.ngroups, hg = blockIdx.y % p.ngroups;
  const int q0 = p.cu_q[b], n = p.cu_q[b + 1] - q0;
  const int r0 = blockIdx.x * kTileQ;
  if (r0 >= n) return;
  const int ctx = p.ctx_lens[b];
  const int nvalid = min(kTileQ, n - r0);
  const int i0 = ctx + r0, i1 = i0 + nvalid - 1;
  const bool qvalid = ln < nvalid;
  const int r = r0 + min(ln, nvalid - 1);
  const int pos = ctx + r;
  const int64_t t = q0 + r;
  const int rep = p.H / p.G;
  const int hloc = hg * 4 + wave;
  const bool active = hloc < rep;
  const int h = g * rep + min(hloc, rep - 1);
  const int D = p.D, Dv = p.Dv, page = p.page, P = p.P, W = p.window;
  const int nkk = D / 16, ndvb = Dv / 16, ldv = Dv + 4;
  const int64_t GD = static_cast<int64_t>(p.G) * D, GDv = static_cast<int64_t>(p.G) * Dv;
  const int32_t* bt = p.block_tables + static_cast<int64_t>(b) * p.bt_stride;

  bf16x4_t qf[kMaxKK];
  {
    const uint16_t* qrow = p.q + (t * p.H + h) * D + 4 * lg;
#pragma unroll
    for (int kk = 0; kk < kMaxKK; ++kk)
      if (kk < nkk) qf[kk] = *reinterpret_cast<const bf16x4_t*>(qrow + 16 * kk);
  }
  f32x4_t acc_o[kMaxDvb];
#pragma unroll
  for (int d = 0; d < kMaxDvb; ++d) acc_o[d] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
  float m = 0.0f, l = p.sink;

  const int nbmax = (P > 0 && i1 - W + 1 > 0) ? (i1 - W + 1) / P : 0;      // pooled blocks the last query sees
  const int jlo = max(0, i0 - W + 1);

  for (int phase = 0; phase < 2; ++phase) {
    const int e_begin = phase == 0 ? 0 : jlo;
    const int e_end = phase == 0 ? nbmax : i1 + 1;                          // entries [e_begin, e_end)
    for (int e0 = e_begin; e0 < e_end; e0 += kTileK) {
      __syncthreads();                                                      // the previous tile's V reads are done
      for (int c = threadIdx.x; c < kTileK * (Dv / 4); c += blockDim.x) {
        const int row = c / (Dv / 4), seg = c - row * (Dv / 4);
        const int e = min(e0 + row, e_end - 1);
        const uint16_t* vrow;
        if (phase == 0) {
          const int pj = (e * P + P - 1) / page;
          vrow = p.vp + (static_cast<int64_t>(bt[pj]) * p.PP + (e - (page * pj) / P)) * GDv + g * Dv;
        } else {
          vrow = p.v_cache + (static_cast<int64_t>(bt[e / page]) * page + e % page) * GDv + g * Dv;
        }
        *reinterpret_cast<uint2*>(vs + row * ldv + seg * 4) = *reinterpret_cast<const uint2*>(vrow + seg * 4);
      }
      __syncthreads();
      if (!active) continue;

      float s[4][4];
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const int e = min(e0 + kb * 16 + ln, e_end - 1);                    // this lane's A row: one key
        const uint16_t* krow;
        if (phase == 0) {
          const int pj = (e * P + P - 1) / page;
          krow = p.kp + (static_cast<int64_t>(bt[pj]) * p.PP + (e - (page * pj) / P)) * GD + g * D;
        } else {
          krow = p.k_cache + (static_cast<int64_t>(bt[e / page]) * page + e % page) * GD + g * D;
        }
        krow += 4 * lg;
        f32x4_t acc = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int kk = 0; kk < kMaxKK; ++kk)
          if (kk < nkk)
            acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(*reinterpret_cast<const bf16x4_t*>(krow + 16 * kk), qf[kk],
                                                            acc, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int ke = e0 + kb * 16 + 4 * lg + i;                         // the key of result row 4*lg + i
          bool vis = ke < e_end;
          if (phase == 0) vis = vis && (ke * P + P - 1 <= pos - W);
          else vis = vis && ke <= pos && pos - ke < W;
          s[kb][i] = vis ? acc[i] * p.scale : -INFINITY;
        }
      }
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[kb][i]);
      mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
      mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
      const float nm = fmaxf(m, mx);
      const float corr = expf(m - nm);
      float rs = 0.0f;
      bf16x4_t pb[4];
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float e = expf(s[kb][i] - nm);                              // exp(-inf) = 0 for what is not seen
          rs += e;
          pb[kb][i] = bf16_bits(e);
        }
      }
      rs += __shfl_xor(rs, 16, kWave);
      rs += __shfl_xor(rs, 32, kWave);
      l = l * corr + rs;
      m = nm;
#pragma unroll
      for (int d = 0; d < kMaxDvb; ++d)
        if (d < ndvb) acc_o[d] *= corr;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        const uint16_t* vt = vs + (kb * 16 + 4 * lg) * ldv + ln;            // V^T fragment: 4 keys of one value column
#pragma unroll
        for (int d = 0; d < kMaxDvb; ++d) {
          if (d < ndvb) {
            bf16x4_t a;
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = static_cast<short>(vt[i * ldv + 16 * d]);
            acc_o[d] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pb[kb], acc_o[d], 0, 0, 0);
          }
        }
      }
    }
  }
  if (!active || !qvalid) return;
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  uint16_t* orow = p.out + (t * p.H + h) * Dv;
  const uint16_t* grow = p.gate != nullptr ? p.gate + t * p.ld_gate + static_cast<int64_t>(h) * Dv : nullptr;
#pragma unroll
  for (int d = 0; d < kMaxDvb; ++d) {
    if (d < ndvb) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int dv = 16 * d + 4 * lg + i;
        float val = acc_o[d][i] * inv;
        if (grow != nullptr) val *= sigmoidf_(__builtin_bit_cast(float, static_cast<uint32_t>(grow[dv]) << 16));
        orow[dv] = static_cast<uint16_t>(bf16_bits(val));
      }
    }
  }
}

}  // namespace lvmix

using namespace lvmix;

extern "C" int lv_window_pool_attn_mfma(const void* q, const void* k_cache, const void* v_cache, const void* kp,
                                        const void* vp, const void* gate, int64_t ld_gate, void* out, const int32_t* cu_q,
                                        const int32_t* ctx_lens, const int32_t* block_tables, int bt_stride, int B,
                                        int max_new_tokens, int H, int G, int D, int Dv, int page, int window, int P,
                                        float scale, int has_sink, void* stream) {
  if (B == 0 || max_new_tokens <= 0) return 0;
  if (!q || !k_cache || !v_cache || !out || !cu_q || !ctx_lens || !block_tables)
    return fail(-1, "lv_window_pool_attn_mfma: null pointer");
  if (P > 0 && (!kp || !vp)) return fail(-1, "lv_window_pool_attn_mfma: pooled blocks without their cache");
  if (B < 0 || H <= 0 || G <= 0 || H % G != 0 || page <= 0 || window <= 0 || bt_stride <= 0)
    return fail(-1, "lv_window_pool_attn_mfma: bad sizes");
  if (D % 16 != 0 || Dv % 16 != 0 || D <= 0 || Dv <= 0 || D > 16 * kMaxKK || Dv > 16 * kMaxDvb)
    return fail(-2, "lv_window_pool_attn_mfma: head sizes %d / %d (multiples of 16 up to 256)", D, Dv);
  if (gate != nullptr && ld_gate < static_cast<int64_t>(H) * Dv) return fail(-1, "lv_window_pool_attn_mfma: gate stride");
  const int rep = H / G;
  const int ngroups = (rep + 3) / 4;
  WindowMfmaParams p{static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(k_cache),
                     static_cast<const uint16_t*>(v_cache), static_cast<const uint16_t*>(kp),
                     static_cast<const uint16_t*>(vp), static_cast<const uint16_t*>(gate), ld_gate,
                     static_cast<uint16_t*>(out), cu_q, ctx_lens, block_tables, bt_stride, H, G, D, Dv, page, window, P,
                     P > 0 ? (page + P - 1) / P : 0, ngroups, scale, has_sink ? 1.0f : 0.0f};
  const size_t shm = static_cast<size_t>(kTileK) * (Dv + 4) * sizeof(uint16_t);
  dim3 grid((max_new_tokens + kTileQ - 1) / kTileQ, G * ngroups, B), block(256);
  window_pool_mfma_kernel<<<grid, block, shm, as_stream(stream)>>>(p);
  return launched("lv_window_pool_attn_mfma");
}
