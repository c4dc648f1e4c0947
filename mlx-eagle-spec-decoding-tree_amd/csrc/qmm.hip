// 4-bit (group 64) quantised matmul for M = 1..32 rows of x, gfx950.
//
//   out[m,n] = fp16( sum_k x[m,k] * (s[n,k/64] * q[n,k] + b[n,k/64]) )
//
// Weight layout is the MLX one: wq[N, K/8] uint32, nibble i of a word is element
// 8*word + i; scales/biases [N, K/64] fp16.  (Reference contract:
// qmm_kernel.py:84-164, kernels/progression/simd_no_swizzle_cast.metal.)
//
// The kernel is a weight streamer.  A wave owns RT tiles of 16 weight rows; per
// 256-wide K chunk every lane issues two 128-bit loads that cover one whole
// quantisation group (64 nibbles = 32 bytes) of one row, so the four lanes that
// share a row read one full 128-byte line.  Nibbles are expanded in registers
// with the fp16 magic-number trick ((w & 0x000f000f) | 0x6400 = 1024 + q,
// (w & 0x00f000f0) | 0x5400 = 64 + q), giving the pairs (q0,q4) (q1,q5) (q2,q6)
// (q3,q7); x is staged through LDS in that same element order, so no shuffle is
// needed.  Products run on v_mfma_f32_16x16x32_f16 with the weight tile as the A
// operand (rows = output features) and the x tile as the B operand (columns =
// rows of x), fp32 accumulation.  K can be split over the waves of a workgroup
// (reduced through LDS) and over workgroups (fp32 partials in a workspace, the
// last workgroup to arrive adds them in a fixed order, so results are
// deterministic).
#include "common.h"

namespace {

constexpr int CHUNK_K = 256;          // K elements per wave step (4 groups)
constexpr int MAX_ROW_BLOCKS = EAGLE_QMM_COUNTER_BYTES / 4;

__device__ inline half2_t as_h2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// (v & mask) | bits in one VALU op.  The compiler splits the two-literal form into
// v_and + v_or; holding `bits` in a VGPR and `mask` in an SGPR makes it encodable.
__device__ inline uint32_t and_or(uint32_t v, uint32_t mask, uint32_t bits) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(bits));
  return r;
}

struct DequantConsts {
  uint32_t magic_lo, magic_hi;   // VGPR copies of 0x64006400 / 0x54005400
};

// 8 nibbles of one packed word -> 8 fp16 weights in the order q0,q4,q1,q5,q2,q6,q3,q7.
__device__ inline half8_t dequant8(uint32_t v, half2_t ss, half2_t bb, const DequantConsts& c) {
  const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
  const half2_t k64 = {(half_t)64.0f, (half_t)64.0f};
  const uint32_t v2 = v >> 8;
  half2_t a0 = as_h2(and_or(v, 0x000f000fu, c.magic_lo)) - k1024;    // 1024 + q  -> q
  half2_t a1 = as_h2(and_or(v, 0x00f000f0u, c.magic_hi)) - k64;      //   64 + q  -> q
  half2_t a2 = as_h2(and_or(v2, 0x000f000fu, c.magic_lo)) - k1024;
  half2_t a3 = as_h2(and_or(v2, 0x00f000f0u, c.magic_hi)) - k64;
  a0 = a0 * ss + bb;
  a1 = a1 * ss + bb;
  a2 = a2 * ss + bb;
  a3 = a3 * ss + bb;
  half8_t r;
  r[0] = a0[0]; r[1] = a0[1]; r[2] = a1[0]; r[3] = a1[1];
  r[4] = a2[0]; r[5] = a2[1]; r[6] = a3[0]; r[7] = a3[1];
  return r;
}

struct WRegs {
  uint4_t lo, hi;   // 64 nibbles of one row
  half2_t ss, bb;   // that group's scale / bias, broadcast
};

template <int NT, int RT, int WR, int WK>
__global__ __launch_bounds__(64 * WR * WK) void qmm_w4g64_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ w,
    const half_t* __restrict__ s, const half_t* __restrict__ b,
    const half_t* __restrict__ bias, half_t* __restrict__ out,
    float* __restrict__ partial, unsigned* __restrict__ counters,
    int M, int N, int K, int stages_per_split) {
  constexpr int NW = WR * WK;
  constexpr int NTHR = 64 * NW;
  constexpr int MP = 16 * NT;
  constexpr int BN = 16 * RT * WR;
  constexpr int STAGE_K = CHUNK_K * WK;
  constexpr int XROW = STAGE_K * 2 + 16;          // bytes; +16 keeps b128 reads conflict free
  constexpr int XBUF = MP * XROW;
  constexpr int VEC_PER_STAGE = MP * STAGE_K / 8; // 16-byte vectors per x stage
  constexpr int VPT = VEC_PER_STAGE / NTHR;
  static_assert(VEC_PER_STAGE % NTHR == 0, "x stage must divide over the threads");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];   // LDS_BYTES, set by launch()
  __shared__ int s_last;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wr = wave % WR;
  const int wk = wave / WR;
  const int r = lane & 15;   // row inside a 16-row tile (A operand) / column m (B operand)
  const int h = lane >> 4;   // which of the chunk's four groups this lane owns
  const int G = K >> 6;
  const int K8 = K >> 3;
  const int nb = blockIdx.x * BN;

  const int nst = (K + STAGE_K - 1) / STAGE_K;
  const int st0 = blockIdx.y * stages_per_split;
  const int st1 = min(st0 + stages_per_split, nst);

  float4_t acc[RT][NT];
#pragma unroll
  for (int i = 0; i < RT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

  size_t wrow[RT], srow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int n = min(nb + (wr * RT + rt) * 16 + r, N - 1);
    wrow[rt] = (size_t)n * K8;
    srow[rt] = (size_t)n * G;
  }

  auto load_w = [&](int st, WRegs (&dst)[RT]) {
    const int g = (st * WK + wk) * 4 + h;
    const bool ok = g < G;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      if (ok) {
        const uint4_t* p = reinterpret_cast<const uint4_t*>(w + wrow[rt] + (size_t)g * 8);
        dst[rt].lo = __builtin_nontemporal_load(p);
        dst[rt].hi = __builtin_nontemporal_load(p + 1);
        const half_t sv = s[srow[rt] + g];
        const half_t bv = b[srow[rt] + g];
        dst[rt].ss = half2_t{sv, sv};
        dst[rt].bb = half2_t{bv, bv};
      } else {
        dst[rt].lo = uint4_t{0, 0, 0, 0};
        dst[rt].hi = uint4_t{0, 0, 0, 0};
        dst[rt].ss = half2_t{(half_t)0.f, (half_t)0.f};
        dst[rt].bb = half2_t{(half_t)0.f, (half_t)0.f};
      }
    }
  };

  auto load_x = [&](int st, half8_t (&dst)[VPT]) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int v = tid + i * NTHR;
      const int row = v / (32 * WK);
      const int col8 = v % (32 * WK);
      const int k = st * STAGE_K + col8 * 8;
      half8_t val = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      if (row < M && k < K) val = *reinterpret_cast<const half8_t*>(x + (size_t)row * K + k);
      dst[i] = val;
    }
  };

  auto store_x = [&](int buf, const half8_t (&src)[VPT]) {
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int v = tid + i * NTHR;
      const int row = v / (32 * WK);
      const int col8 = v % (32 * WK);
      const half8_t a = src[i];
      half8_t p;   // element order matching dequant8: 0,4,1,5,2,6,3,7
      p[0] = a[0]; p[1] = a[4]; p[2] = a[1]; p[3] = a[5];
      p[4] = a[2]; p[5] = a[6]; p[6] = a[3]; p[7] = a[7];
      *reinterpret_cast<half8_t*>(lds + buf * XBUF + row * XROW + col8 * 16) = p;
    }
  };

  DequantConsts dq;
  asm volatile("v_mov_b32 %0, 0x64006400" : "=v"(dq.magic_lo));
  asm volatile("v_mov_b32 %0, 0x54005400" : "=v"(dq.magic_hi));
  WRegs wcur[RT], wnext[RT];
  half8_t xreg[VPT];

  if (st0 < st1) {
    load_x(st0, xreg);
    load_w(st0, wcur);
    store_x(0, xreg);
  }
  __syncthreads();

  for (int st = st0; st < st1; ++st) {
    const int buf = (st - st0) & 1;
    const bool more = (st + 1) < st1;
    if (more) {
      load_w(st + 1, wnext);
      load_x(st + 1, xreg);
    }
    const unsigned char* xb = lds + buf * XBUF + r * XROW + wk * (CHUNK_K * 2) + h * 128;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      half8_t bx[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        bx[nt] = *reinterpret_cast<const half8_t*>(xb + nt * 16 * XROW + t * 16);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const uint32_t word = (t < 4) ? wcur[rt].lo[t & 3] : wcur[rt].hi[t & 3];
        const half8_t a = dequant8(word, wcur[rt].ss, wcur[rt].bb, dq);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          acc[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bx[nt], acc[rt][nt], 0, 0, 0);
      }
    }
    if (more) store_x(buf ^ 1, xreg);
    __syncthreads();
    if (more) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) wcur[rt] = wnext[rt];
    }
  }

  // ---- reduce the K split held by the waves of this workgroup --------------------
  if (WK > 1) {
    float4_t* red = reinterpret_cast<float4_t*>(lds);
    if (wk > 0) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          red[((((wk - 1) * WR + wr) * RT + rt) * NT + nt) * 64 + lane] = acc[rt][nt];
    }
    __syncthreads();
    if (wk == 0) {
#pragma unroll
      for (int k2 = 1; k2 < WK; ++k2)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
            acc[rt][nt] += red[((((k2 - 1) * WR + wr) * RT + rt) * NT + nt) * 64 + lane];
    }
  }

  // ---- reduce the K split over workgroups ------------------------------------------
  const int nsplit = gridDim.y;
  if (nsplit > 1) {
    float4_t* pbase = reinterpret_cast<float4_t*>(partial) +
                      (size_t)blockIdx.x * nsplit * (WR * RT * NT * 64);
    if (wk == 0) {
      float4_t* mine = pbase + (size_t)blockIdx.y * (WR * RT * NT * 64);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          mine[((wr * RT + rt) * NT + nt) * 64 + lane] = acc[rt][nt];
    }
    __threadfence();
    __syncthreads();
    if (tid == 0) {
      const unsigned old = atomicAdd(&counters[blockIdx.x], 1u);
      s_last = (old == (unsigned)(nsplit - 1));
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();
    if (wk == 0) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          float4_t sum = float4_t{0.f, 0.f, 0.f, 0.f};
          for (int sp = 0; sp < nsplit; ++sp)
            sum += __builtin_nontemporal_load(
                pbase + (size_t)sp * (WR * RT * NT * 64) + ((wr * RT + rt) * NT + nt) * 64 + lane);
          acc[rt][nt] = sum;
        }
    }
    if (tid == 0) counters[blockIdx.x] = 0u;
  }

  // ---- epilogue: lane holds out[m = 16 nt + r][n = tile + 4 h + i], i = 0..3 ---------
  if (wk == 0) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int n0 = nb + (wr * RT + rt) * 16 + 4 * h;
      if (n0 >= N) continue;   // N % 8 == 0, so a group of four is all in or all out
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const int m = nt * 16 + r;
        if (m >= M) continue;
        half4_t o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          half_t v = (half_t)acc[rt][nt][i];
          if (bias) v = (half_t)((float)v + (float)bias[n0 + i]);
          o[i] = v;
        }
        *reinterpret_cast<half4_t*>(out + (size_t)m * N + n0) = o;
      }
    }
  }
}

struct Variant {
  const char* name;
  int rt, wr, wk;
};
// Tile shapes compiled in.  BN = 16*rt*wr output rows per workgroup.
constexpr Variant kVariants[] = {
    {"bn64_w4x1", 1, 4, 1},
    {"bn128_w4x1", 2, 4, 1},
    {"bn32_w2x2", 1, 2, 2},
    {"bn16_w1x4", 1, 1, 4},
    {"bn64_w4x2", 1, 4, 2},
    {"bn32_w2x4", 1, 2, 4},
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

template <int NT, int RT, int WR, int WK>
constexpr int lds_bytes() {
  constexpr int xbuf = 2 * (16 * NT) * (CHUNK_K * WK * 2 + 16);
  constexpr int red = (WK > 1) ? (WK - 1) * WR * RT * NT * 64 * 16 : 0;
  return xbuf > red ? xbuf : red;
}

template <int NT, int RT, int WR, int WK>
void launch(const void* x, const uint32_t* wq, const void* s, const void* b, const void* bias,
            void* out, float* partial, unsigned* counters, int M, int N, int K, int splits,
            hipStream_t stream) {
  constexpr int BN = 16 * RT * WR;
  constexpr int STAGE_K = CHUNK_K * WK;
  const int nst = (K + STAGE_K - 1) / STAGE_K;
  const int sps = (nst + splits - 1) / splits;
  const int eff_splits = (nst + sps - 1) / sps;
  dim3 grid((N + BN - 1) / BN, eff_splits);
  constexpr int lds = lds_bytes<NT, RT, WR, WK>();
  static bool attr_set = false;   // more than 64 KB of LDS needs an explicit opt-in, once
  if (lds > 65536 && !attr_set) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&qmm_w4g64_kernel<NT, RT, WR, WK>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    attr_set = true;
  }
  hipLaunchKernelGGL((qmm_w4g64_kernel<NT, RT, WR, WK>), grid, dim3(64 * WR * WK), lds, stream,
                     (const half_t*)x, wq, (const half_t*)s, (const half_t*)b,
                     (const half_t*)bias, (half_t*)out, partial, counters, M, N, K, sps);
}

template <int NT>
void dispatch(int variant, const void* x, const uint32_t* wq, const void* s, const void* b,
              const void* bias, void* out, float* partial, unsigned* counters, int M, int N,
              int K, int splits, hipStream_t stream) {
  switch (variant) {
    case 0: launch<NT, 1, 4, 1>(x, wq, s, b, bias, out, partial, counters, M, N, K, splits, stream); break;
    case 1: launch<NT, 2, 4, 1>(x, wq, s, b, bias, out, partial, counters, M, N, K, splits, stream); break;
    case 2: launch<NT, 1, 2, 2>(x, wq, s, b, bias, out, partial, counters, M, N, K, splits, stream); break;
    case 3: launch<NT, 1, 1, 4>(x, wq, s, b, bias, out, partial, counters, M, N, K, splits, stream); break;
    case 4: launch<NT, 1, 4, 2>(x, wq, s, b, bias, out, partial, counters, M, N, K, splits, stream); break;
    default: launch<NT, 1, 2, 4>(x, wq, s, b, bias, out, partial, counters, M, N, K, splits, stream); break;
  }
}

int block_rows(int variant) { return 16 * kVariants[variant].rt * kVariants[variant].wr; }

// Largest split count the workspace formula and the counters allow for a variant.
int max_splits(int variant, int N, int K) {
  const int stage_k = CHUNK_K * kVariants[variant].wk;
  const int nst = (K + stage_k - 1) / stage_k;
  const int rb = (N + block_rows(variant) - 1) / block_rows(variant);
  if (rb > MAX_ROW_BLOCKS) return 1;
  return nst < 16 ? nst : 16;
}

// Heuristic launch shape.  Aim for at least two workgroups per compute unit, prefer
// wide row blocks (x is re-read once per row block) and keep the fp32 partial traffic
// of a K split small next to the weight bytes.
void choose(int M, int N, int K, int* variant, int* splits) {
  const int target_wgs = 512;
  int v;
  if (N >= 128 * target_wgs) v = 1;
  else if (N >= 64 * target_wgs) v = 0;
  else if (N >= 32 * (target_wgs / 2)) v = 2;
  else v = 3;
  const int rb = (N + block_rows(v) - 1) / block_rows(v);
  int sp = 1;
  if (rb < target_wgs) {
    sp = (target_wgs + rb - 1) / rb;
    const int mp = M <= 16 ? 16 : 32;
    int cap = K / (48 * mp);          // partial bytes <= ~1/3 of the weight bytes
    if (cap < 1) cap = 1;
    if (sp > cap) sp = cap;
    const int ms = max_splits(v, N, K);
    if (sp > ms) sp = ms;
  }
  *variant = v;
  *splits = sp;
}

size_t partial_bytes(int variant, int splits, int M, int N) {
  if (splits <= 1) return 0;
  const int bn = block_rows(variant);
  const size_t rb = ((size_t)N + bn - 1) / bn;
  const size_t mp = M <= 16 ? 16 : 32;
  return rb * splits * bn * mp * sizeof(float);
}

int validate(const void* x, const uint32_t* wq, const void* s, const void* b, const void* bias,
             void* out, int M, int N, int K) {
  if (!x || !wq || !s || !b || !out) return EAGLE_ERR_NULL;
  if (M < 1 || M > EAGLE_MAX_M || N < 8 || (N % 8) != 0 || K < 64 || (K % 64) != 0)
    return EAGLE_ERR_SHAPE;
  if (!eagle_aligned16(x) || !eagle_aligned16(wq) || !eagle_aligned16(out) ||
      (reinterpret_cast<uintptr_t>(s) & 1u) || (reinterpret_cast<uintptr_t>(b) & 1u) ||
      (bias && (reinterpret_cast<uintptr_t>(bias) & 1u)))
    return EAGLE_ERR_ALIGN;
  // rows of x and wq must keep 16-byte alignment
  if ((K % 8) != 0) return EAGLE_ERR_SHAPE;
  return EAGLE_OK;
}

}  // namespace

EAGLE_EXPORT size_t eagle_qmm_workspace_bytes_cfg(int M, int N, int K, int variant, int splits) {
  if (M < 1 || N < 1 || K < 64 || variant >= kNumVariants) return 0;
  if (variant < 0) choose(M, N, K, &variant, &splits);
  const int ms = max_splits(variant, N, K);
  if (splits > ms) splits = ms;
  return (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(variant, splits, M, N);
}

EAGLE_EXPORT size_t eagle_qmm_workspace_bytes(int M, int N, int K) {
  return eagle_qmm_workspace_bytes_cfg(M, N, K, -1, 0);
}

EAGLE_EXPORT int eagle_qmm_num_variants(void) { return kNumVariants; }

EAGLE_EXPORT const char* eagle_qmm_variant_name(int variant) {
  if (variant < 0 || variant >= kNumVariants) return "heuristic";
  return kVariants[variant].name;
}

EAGLE_EXPORT int eagle_qmm_w4g64_f16_cfg(const void* x, const uint32_t* wq, const void* scales,
                                         const void* biases, const void* bias, void* out, int M,
                                         int N, int K, int variant, int splits, void* workspace,
                                         size_t workspace_bytes, eagle_stream_t stream) {
  const int rc = validate(x, wq, scales, biases, bias, out, M, N, K);
  if (rc != EAGLE_OK) return rc;
  if (variant >= kNumVariants) return EAGLE_ERR_SHAPE;
  if (variant < 0) choose(M, N, K, &variant, &splits);
  if (splits < 1) splits = 1;
  const int ms = max_splits(variant, N, K);
  if (splits > ms) splits = ms;
  float* partial = nullptr;
  unsigned* counters = nullptr;
  if (splits > 1) {
    if (!workspace || !eagle_aligned16(workspace) ||
        workspace_bytes < (size_t)EAGLE_QMM_COUNTER_BYTES + partial_bytes(variant, splits, M, N))
      return EAGLE_ERR_WORKSPACE;
    counters = reinterpret_cast<unsigned*>(workspace);
    partial = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) +
                                       EAGLE_QMM_COUNTER_BYTES);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (M <= 16)
    dispatch<1>(variant, x, wq, scales, biases, bias, out, partial, counters, M, N, K, splits, st);
  else
    dispatch<2>(variant, x, wq, scales, biases, bias, out, partial, counters, M, N, K, splits, st);
  return eagle_launch_status();
}

EAGLE_EXPORT int eagle_qmm_w4g64_f16(const void* x, const uint32_t* wq, const void* scales,
                                     const void* biases, const void* bias, void* out, int M,
                                     int N, int K, int group_size, int bits, void* workspace,
                                     size_t workspace_bytes, eagle_stream_t stream) {
  if (group_size != 64 || bits != 4) return EAGLE_ERR_UNSUPPORTED;
  return eagle_qmm_w4g64_f16_cfg(x, wq, scales, biases, bias, out, M, N, K, -1, 0, workspace,
                                 workspace_bytes, stream);
}
