// Flash attention forward on the vector ALUs: the fp32 path (parity budget 1e-5, which rules
// out half-precision matrix cores) and the fallback for head dims the MFMA kernels do not tile
// (anything that is not a multiple of 8, and 129 .. 256, the range decode attention accepts too).
//
// Same recurrence as flash_attn_cpu (reference src/Execution.jl:453-479), evaluated a tile of
// 32 keys at a time: m' = max(m, tile max), o = o*exp(m-m') + sum_j exp(s_j-m') v_j,
// l = l*exp(m-m') + sum_j exp(s_j-m'), out = o / l.
//
// Work split: one workgroup = 64 query rows of one (b, hq); 4 lanes share a row, each holding a
// quarter of q and of the output accumulator in registers. K/V tiles are staged in LDS as fp32
// and read as float4 (the 16 row-groups of a wave read the same address -> LDS broadcast).
#include "common.hpp"
#include "dtypes.hpp"
#include "rope.hpp"

namespace lmh {
namespace {

constexpr int kRowsPerWg = 64;
constexpr int kLanesPerRow = 4;
// keys per staged tile: 32; 16 for head dims above 128, whose fp32 tiles would not fit the 64 KB of static LDS
template <int DP> constexpr int keys_per_tile() { return DP > 128 ? 16 : 32; }

template <typename E, int DP>
__global__ __launch_bounds__(256) void prefill_valu_kernel(PrefillArgs a) {
  request_args(a);
  using raw = typename E::raw;
  constexpr int NCH = DP / 16;  // float4 chunks per lane
  constexpr int kKeysPerTile = keys_per_tile<DP>();
  __shared__ float4 Ks[kKeysPerTile][DP / 4];
  __shared__ float4 Vs[kKeysPerTile][DP / 4];

  const int tid = threadIdx.x;
  const int t = tid & 3;
  const int row_in_wg = tid >> 2;
  const int b = blockIdx.z, hq = blockIdx.y;
  const int kvh = kv_head_of(hq, a.Hq, a.Hkv, a.head_map);
  const int q0 = blockIdx.x * kRowsPerWg;
  const int qi = q0 + row_in_wg;
  const bool row_valid = qi < a.Sq;
  const int D = a.D;

  int n_keys = a.kv_len ? a.kv_len[b] : a.Sk;
  n_keys = min(max(n_keys, 0), a.Sk);
  int k_end = n_keys;
  if (a.causal) k_end = min(k_end, q0 + kRowsPerWg);  // no row of this workgroup sees further

  const raw *qp = reinterpret_cast<const raw *>(a.q) + b * a.qs[0] + hq * a.qs[1] + (int64_t)qi * a.qs[2];
  const raw *kp = reinterpret_cast<const raw *>(a.k) + b * a.ks[0] + kvh * a.ks[1];
  const raw *vp = reinterpret_cast<const raw *>(a.v) + b * a.vs[0] + kvh * a.vs[1];

  float4 qf[NCH], of[NCH];
#pragma unroll
  for (int c = 0; c < NCH; c++) {
    float tmp[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      int d = (c * 4 + t) * 4 + e;
      tmp[e] = (row_valid && d < D) ? E::ld(qp[d]) : 0.f;
      // rotary embedding on the way in (PrefillArgs::q_rope), rounded to the element type as lmh_rope stores it
      if (a.q_rope && row_valid && d < D)
        tmp[e] = E::ld(E::st(rope_element(qp, d, D, (float)((a.q_pos0 ? a.q_pos0[b] : a.q_prev_seq) + qi), a.q_log2_base,
                                          a.q_interleaved != 0, [](raw x) { return E::ld(x); })));
    }
    qf[c] = make_float4(tmp[0], tmp[1], tmp[2], tmp[3]);
    of[c] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float m_i = -INFINITY, l_i = 0.f;

  for (int k0 = 0; k0 < k_end; k0 += kKeysPerTile) {
    __syncthreads();  // previous tile fully consumed
    for (int idx = tid; idx < kKeysPerTile * DP; idx += 256) {
      int r = idx / DP, d = idx % DP;
      int key = k0 + r;
      float kx = 0.f, vx = 0.f;
      if (key < n_keys && d < D) {
        kx = E::ld(kp[(int64_t)key * a.ks[2] + d]);
        vx = E::ld(vp[(int64_t)key * a.vs[2] + d]);
      }
      reinterpret_cast<float *>(&Ks[r][0])[d] = kx;
      reinterpret_cast<float *>(&Vs[r][0])[d] = vx;
    }
    __syncthreads();

    float s[kKeysPerTile];
    float tile_max = -INFINITY;
#pragma unroll
    for (int j = 0; j < kKeysPerTile; j++) {
      float acc = 0.f;
#pragma unroll
      for (int c = 0; c < NCH; c++) {
        float4 kk = Ks[j][c * 4 + t];
        acc += qf[c].x * kk.x;
        acc += qf[c].y * kk.y;
        acc += qf[c].z * kk.z;
        acc += qf[c].w * kk.w;
      }
      acc += __shfl_xor(acc, 1);
      acc += __shfl_xor(acc, 2);
      int key = k0 + j;
      bool keep = key < n_keys && !(a.causal && key > qi);
      s[j] = keep ? acc * a.scale : -INFINITY;
      tile_max = fmaxf(tile_max, s[j]);
    }
    float m_next = fmaxf(m_i, tile_max);
    float alpha = (m_i == -INFINITY) ? 0.f : expf(m_i - m_next);
    l_i *= alpha;
#pragma unroll
    for (int c = 0; c < NCH; c++) {
      of[c].x *= alpha; of[c].y *= alpha; of[c].z *= alpha; of[c].w *= alpha;
    }
#pragma unroll
    for (int j = 0; j < kKeysPerTile; j++) {
      float p = (s[j] == -INFINITY) ? 0.f : expf(s[j] - m_next);
      l_i += p;
#pragma unroll
      for (int c = 0; c < NCH; c++) {
        float4 vv = Vs[j][c * 4 + t];
        of[c].x += p * vv.x; of[c].y += p * vv.y; of[c].z += p * vv.z; of[c].w += p * vv.w;
      }
    }
    m_i = m_next;
  }

  if (row_valid) {
    const int64_t off = b * a.os[0] + hq * a.os[1] + (int64_t)qi * a.os[2];
    raw *op = reinterpret_cast<raw *>(a.out) + off;
    float *op32 = reinterpret_cast<float *>(a.out) + off;
    float inv = l_i > 0.f ? 1.f / l_i : 0.f;  // a row with no visible key (kv_len[b] == 0) is written as zeros
#pragma unroll
    for (int c = 0; c < NCH; c++) {
      float tmp[4] = {of[c].x, of[c].y, of[c].z, of[c].w};
#pragma unroll
      for (int e = 0; e < 4; e++) {
        int d = (c * 4 + t) * 4 + e;
        if (d < D) {
          if (a.out_f32) op32[d] = tmp[e] * inv;
          else op[d] = E::st(tmp[e] * inv);
        }
      }
    }
  }
}

template <typename E>
int launch_for_dtype(const PrefillArgs &a, hipStream_t stream) {
  dim3 grid((a.Sq + kRowsPerWg - 1) / kRowsPerWg, a.Hq, a.B), block(256);
  if (a.D <= 256 && plan_only("prefill_valu_kernel<%s, head dim %d padded to %d> workgroups=%u", E::kName, a.D,
                              a.D <= 16 ? 16 : a.D <= 32 ? 32 : a.D <= 64 ? 64 : a.D <= 96 ? 96 : a.D <= 128 ? 128 : a.D <= 192 ? 192 : 256,
                              grid.x * grid.y * grid.z))
    return LMH_OK;
  if (a.D <= 16) hipLaunchKernelGGL((prefill_valu_kernel<E, 16>), grid, block, 0, stream, a);
  else if (a.D <= 32) hipLaunchKernelGGL((prefill_valu_kernel<E, 32>), grid, block, 0, stream, a);
  else if (a.D <= 64) hipLaunchKernelGGL((prefill_valu_kernel<E, 64>), grid, block, 0, stream, a);
  else if (a.D <= 96) hipLaunchKernelGGL((prefill_valu_kernel<E, 96>), grid, block, 0, stream, a);
  else if (a.D <= 128) hipLaunchKernelGGL((prefill_valu_kernel<E, 128>), grid, block, 0, stream, a);
  else if (a.D <= 192) hipLaunchKernelGGL((prefill_valu_kernel<E, 192>), grid, block, 0, stream, a);
  else if (a.D <= 256) hipLaunchKernelGGL((prefill_valu_kernel<E, 256>), grid, block, 0, stream, a);
  else return fail(LMH_E_UNSUPPORTED, "flash attention: head dim %d > 256 is not supported", a.D);
  LMH_HIP_TRY(hipGetLastError());
  return LMH_OK;
}

}  // namespace

int launch_prefill_valu(const PrefillArgs &a, int dtype, hipStream_t stream) {
  switch (dtype) {
    case LMH_F32: return launch_for_dtype<F32>(a, stream);
    case LMH_F16: return launch_for_dtype<F16>(a, stream);
    case LMH_BF16: return launch_for_dtype<BF16>(a, stream);
  }
  return fail(LMH_E_UNSUPPORTED, "flash attention: unknown dtype %d", dtype);
}

}  // namespace lmh
