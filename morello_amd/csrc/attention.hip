// Fused Matmul -> Softmax -> Matmul for bf16 inputs (the attention-shaped Compose of
// morello/examples/matmul_chain.rs:26-57; semantics morello/src/verification.rs:225-286):
//     S = Q . KT        [m, n2]  f32
//     P = softmax(S)    row-wise over n2, f32
//     out = P . V       [m, n]   f32
// with no scale and no mask, one independent problem per batch entry.
//
// The reference materialises S and P in memory between three loop nests
// (matmul_chain.rs:60-81).  Here a workgroup owns 128 query rows of one batch entry and
// streams blocks of 64 keys: S^T = K.Q^T is formed on the bf16 MFMA, folded into a running
// (max, denominator) per query with the online update of morello/src/spec.rs:96-123
// (new = max(old, x); d = d*exp(old-new) + exp(x-new)), and P^T (rounded to bf16, the one
// deviation from the f32 closed form; at most 2^-9 relative per element) feeds the second
// MFMA as O^T += V^T.P^T.  S and P never reach HBM: traffic is Q, K, V once and the
// output once.
//
// Both products are formed transposed so that a lane owns one query column: the running
// max, the denominator and the rescale factor are per-lane scalars, and a row reduction is
// 32 in-register values plus one cross-lane exchange.
#include "kernels.h"

namespace mrl {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) v4s lds_v4s;

constexpr int D = 128;        // head dim of both products (k and n of the Compose)
constexpr int BQ = 128;       // queries per workgroup (4 waves x 32)
constexpr int BKV = 64;       // keys per block
constexpr int K_ROW = D * 2;          // 256 B, 16-byte chunks XOR-swizzled by (row & 15)
constexpr int V_ROW = D * 2 + 64;     // 320 B: 4 rows x 64 B cover all 64 banks
constexpr int K_BYTES = BKV * K_ROW, V_BYTES = BKV * V_ROW;

__device__ inline v2i read_tr16(const uint8_t *p) {
  const v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s *)p);
  return __builtin_bit_cast(v2i, r);
}

__global__ __launch_bounds__(256) void k_attn(AttnArgs p) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[K_BYTES + V_BYTES];
  uint8_t *lk = lds, *lv = lds + K_BYTES;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lq = lane & 31, lg = lane >> 5;
  const int64_t head = blockIdx.y;
  const int q0 = blockIdx.x * BQ + wave * 32;

  const uint8_t *Q = (const uint8_t *)p.q + (head * p.m + q0 + lq) * int64_t(D) * 2;
  const uint8_t *K = (const uint8_t *)p.kt + head * int64_t(p.n2) * D * 2;
  const uint8_t *V = (const uint8_t *)p.v + head * int64_t(p.n2) * D * 2;

  // Q^T operand: lane (query lq, half lg) holds d = 16*step + 8*lg .. +7.
  v4i qf[D / 16];
#pragma unroll
  for (int s = 0; s < D / 16; s++) qf[s] = *(const v4i *)(Q + s * 32 + lg * 16);

  // Staging: 1024 16-byte chunks each for K and V per block, 4 per thread.
  int src_off[4], k_dst[4], v_dst[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int id = tid + i * 256, row = id >> 4, ch = id & 15;
    src_off[i] = row * (D * 2) + ch * 16;
    k_dst[i] = row * K_ROW + ((ch ^ (row & 15)) << 4);
    v_dst[i] = row * V_ROW + ch * 16;
  }
  v4i kreg[4], vreg[4];
  auto load_block = [&](int kb) {
    const int64_t base = int64_t(kb) * BKV * D * 2;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      kreg[i] = *(const v4i *)(K + base + src_off[i]);
      vreg[i] = *(const v4i *)(V + base + src_off[i]);
    }
  };

  v16f o[D / 32];
#pragma unroll
  for (int t = 0; t < D / 32; t++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[t][r] = 0.0f;
  float m_run = -3.40282347e+38f, l_run = 0.0f;  // l_run: this lane's share of the denominator

  const int nblocks = int(p.n2 / BKV);
  load_block(0);
  for (int kb = 0; kb < nblocks; kb++) {
    __syncthreads();  // everyone is done reading the previous block
#pragma unroll
    for (int i = 0; i < 4; i++) {
      *(v4i *)(lk + k_dst[i]) = kreg[i];
      *(v4i *)(lv + v_dst[i]) = vreg[i];
    }
    __syncthreads();
    if (kb + 1 < nblocks) load_block(kb + 1);

    // S^T tiles: s[kt][r] is key kt*32 + 8*(r/4) + 4*lg + r%4, query lq.
    v16f s[BKV / 32];
#pragma unroll
    for (int kt = 0; kt < BKV / 32; kt++) {
#pragma unroll
      for (int r = 0; r < 16; r++) s[kt][r] = 0.0f;
      const int row = kt * 32 + lq;
#pragma unroll
      for (int st = 0; st < D / 16; st++) {
        const v4i kf = *(const v4i *)(lk + row * K_ROW + (((2 * st + lg) ^ (row & 15)) << 4));
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, kf),
                                                        __builtin_bit_cast(v8bf, qf[st]), s[kt], 0, 0, 0);
      }
    }
    // Online softmax update for this lane's query.
    float mx = s[0][0];
#pragma unroll
    for (int kt = 0; kt < BKV / 32; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[kt][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __expf(m_run - m_new);
    m_run = m_new;
    float psum = 0.0f;
    v8bf pb[BKV / 16];
#pragma unroll
    for (int kt = 0; kt < BKV / 32; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float e = __expf(s[kt][r] - m_new);
        psum += e;
        pb[kt * 2 + r / 8][r % 8] = (__bf16)e;
      }
    l_run = l_run * alpha + psum;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int t = 0; t < D / 32; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[t][r] *= alpha;
    }
    // O^T += V^T . P^T.  Key step u covers keys 16u + {4*lg + c, 8 + 4*lg + c}, c = 0..3,
    // which is the order P^T's registers already have.
#pragma unroll
    for (int u = 0; u < BKV / 16; u++) {
      const int key0 = 16 * u + 4 * lg + ((lane & 15) >> 2);
#pragma unroll
      for (int t = 0; t < D / 32; t++) {
        const int col = t * 32 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
        const v2i lo = read_tr16(lv + key0 * V_ROW + col * 2);
        const v2i hi = read_tr16(lv + (key0 + 8) * V_ROW + col * 2);
        const v4i vf = v4i{lo[0], lo[1], hi[0], hi[1]};
        o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, vf), pb[u], o[t], 0, 0, 0);
      }
    }
  }

  const float denom = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / denom;
  float *out = p.out + (head * p.m + q0 + lq) * int64_t(D);
#pragma unroll
  for (int t = 0; t < D / 32; t++)
#pragma unroll
    for (int a = 0; a < 4; a++) {
      float4 v;
      v.x = o[t][4 * a + 0] * inv, v.y = o[t][4 * a + 1] * inv;
      v.z = o[t][4 * a + 2] * inv, v.w = o[t][4 * a + 3] * inv;
      *(float4 *)(out + t * 32 + 8 * a + 4 * lg) = v;
    }
}

}  // namespace

bool attn_applicable(const AttnArgs &a) {
  auto al16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  return a.k == D && a.n == D && a.m % BQ == 0 && a.n2 % BKV == 0 && a.m && a.n2 && a.b &&
         a.b <= 65535 && al16(a.q) && al16(a.kt) && al16(a.v) && al16(a.out);
}

hipError_t launch_attn(const AttnArgs &a, hipStream_t stream) {
  hipLaunchKernelGGL(k_attn, dim3(a.m / BQ, a.b), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace mrl
