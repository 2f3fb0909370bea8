// softmax(alpha * Q K) V for a batch of heads in one launch.
//
// The reference has no such operator: it runs MatMul, Mul, Softmax, MatMul as four
// nodes (src/descriptor_runner/operators/cpu/operators/standard/matmul.ts:11-111,
// softmax.ts:34-57).  This kernel produces what that chain produces, with the same
// rounding points: scores rounded to fp32 after the scale, the row maximum subtracted,
// e^x in fp32, the fp32 row sum, every e scaled by the sum's reciprocal (as the
// Softmax kernel of this library does), and the second product accumulated in fp32.
// Only the order of the additions inside the two products and the row sum differs.
//
// A workgroup of eight or sixteen wavefronts owns 32 query rows of one head:
//   1. scores: each wavefront takes 32-key column blocks in turn
//      (v_mfma_f32_32x32x2_f32 over the head dimension) and writes alpha * S to LDS,
//      the whole 32 x keys block (keys <= 1024: 129 KB of the CU's 160 KB);
//   2. softmax: four (two) rows per wavefront, in place in LDS;
//   3. output: the keys are cut across the wavefronts in blocks of 32, each wavefront
//      accumulates its share of P V on the matrix cores, and the partial 32 x HD
//      blocks are added in wavefront order through LDS.
// Within a block of 32 keys (or of the head dimension) the two halves of a wavefront
// take the lower and the upper 16 indices, so that a lane reads 16 contiguous floats
// of Q, K and P (16-byte loads) where the MFMA's natural order would interleave them.
#include <math.h>

#include "common.h"
#include "rowmath.h"

namespace {

using namespace wdh::rowmath;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int ATT_ROWS = 32;
constexpr int ATT_MAX_KEYS = 1024;

struct AttParams {
  const float *Q, *K, *V;
  float *Y;
  int tq, tk;
  int pitch;        // floats per LDS row: >= keys rounded up to 32, pitch/4 odd
  int row_blocks;   // ceil(tq / 32)
  long long sQb, sQi, sKb, sKj, sVb, sVj, sYb, sYi;
  float alpha;
};

// ATT_WAVES wavefronts per workgroup: 16 for a head dimension of 32 (every phase is a chain of
// dependent steps per wavefront; twice the wavefronts halve each chain), 8 where a wavefront's
// registers hold less of K and V.
template <int HD, int ATT_WAVES>
__global__ __launch_bounds__(64 * ATT_WAVES) void attention_rows_kernel(AttParams p) {
  static_assert(HD % 32 == 0 && HD >= 32 && HD <= 128, "head dimension");
  static_assert(ATT_WAVES == 8 || ATT_WAVES == 16, "32 rows and 32 key blocks are dealt over the wavefronts");
  constexpr int HALF = HD / 2;   // head-dimension indices per half wavefront
  constexpr int NB = HD / 32;    // 32-column blocks of the output
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 31, half = lane >> 5;
  const int b = blockIdx.x / p.row_blocks;
  const int row0 = (blockIdx.x - b * p.row_blocks) * ATT_ROWS;
  const float *Q = p.Q + (long long)b * p.sQb;
  const float *K = p.K + (long long)b * p.sKb;
  const float *V = p.V + (long long)b * p.sVb;
  const int ncb = (p.tk + 31) >> 5;  // blocks of 32 keys

  // At most 1024 keys are 32 blocks of 32: four (two) per wavefront.  Each phase issues the loads
  // of all four before the first use, so a wavefront waits for memory once per phase.
  constexpr int PER_WAVE = ATT_MAX_KEYS / 32 / ATT_WAVES;

  // Every value of V this wavefront will need in step 3 is requested before step 1, so the
  // loads travel while the scores are computed (64 registers per 32 columns of V).
  float vb[NB == 1 ? PER_WAVE : 1][NB][16];
  if constexpr (NB == 1) {
#pragma unroll
    for (int it = 0; it < PER_WAVE; it++) {
      const int key0 = (wave + ATT_WAVES * it) * 32 + 16 * half;
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int s = 0; s < 16; s++) {
          const int key = key0 + s;
          const float t = V[(long long)(key < p.tk ? key : p.tk - 1) * p.sVj + nb * 32 + li];
          vb[it][nb][s] = key < p.tk ? t : 0.0f;  // (P is 0 there; this keeps an inf or NaN of V out)
        }
    }
  }

  // ---- 1. scores -------------------------------------------------------------------
  {
    float qa[HALF];
    const int qrow = row0 + li < p.tq ? row0 + li : p.tq - 1;  // rows past the end are never stored
    const float *q = Q + (long long)qrow * p.sQi + HALF * half;
#pragma unroll
    for (int c = 0; c < HALF / 4; c++) {
      const f32x4 t = *reinterpret_cast<const f32x4 *>(q + 4 * c);
      qa[4 * c] = t.x; qa[4 * c + 1] = t.y; qa[4 * c + 2] = t.z; qa[4 * c + 3] = t.w;
    }
    f32x4 kb[PER_WAVE][HALF / 4];
#pragma unroll
    for (int it = 0; it < PER_WAVE; it++) {
      const int key = (wave + ATT_WAVES * it) * 32 + li;
      const float *k = K + (long long)(key < p.tk ? key : p.tk - 1) * p.sKj + HALF * half;
#pragma unroll
      for (int c = 0; c < HALF / 4; c++) kb[it][c] = *reinterpret_cast<const f32x4 *>(k + 4 * c);
    }
#pragma unroll
    for (int it = 0; it < PER_WAVE; it++) {
      const int cb = wave + ATT_WAVES * it;
      if (cb >= ncb) break;
      const int key = cb * 32 + li;
      const bool key_ok = key < p.tk;
      f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < HALF; s++)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[s], kb[it][s >> 2][s & 3], acc, 0, 0, 0);
      // lane holds column li, rows 8*(r/4) + 4*half + r%4; keys past the end count as -inf
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int row = 8 * (r >> 2) + 4 * half + (r & 3);
        lds[row * p.pitch + key] = key_ok ? p.alpha * acc[r] : -INFINITY;
      }
    }
  }
  __syncthreads();

  // ---- 2. softmax over each row, in place (softmax.ts:34-57) ------------------------
  // The wavefront's four (two) rows are taken through every step together.
  {
    constexpr int RPW = ATT_ROWS / ATT_WAVES;
    const int ncols = ncb * 32;  // a multiple of 4; at most 1024: four 16-byte pieces per lane
    const float ninf = -INFINITY;
    f32x4 v[RPW][4];
    float mx[RPW], sum[RPW];
#pragma unroll
    for (int j = 0; j < RPW; j++) {
      const float *srow = lds + (wave + ATT_WAVES * j) * p.pitch;
      mx[j] = ninf;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int c = 4 * lane + 256 * i;
        v[j][i] = c < ncols ? *reinterpret_cast<const f32x4 *>(srow + c) : f32x4{ninf, ninf, ninf, ninf};
#pragma unroll
        for (int e = 0; e < 4; e++) mx[j] = fmaxf(mx[j], v[j][i][e]);  // fmaxf skips NaN, like `if (v > max)`
      }
    }
#pragma unroll
    for (int j = 0; j < RPW; j++) mx[j] = wave_max(mx[j]);
#pragma unroll
    for (int j = 0; j < RPW; j++) {
      sum[j] = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const float ex = 4 * lane + 256 * i + e < p.tk ? exp_f32(v[j][i][e] - mx[j]) : 0.0f;
          v[j][i][e] = ex;
          sum[j] += ex;
        }
    }
#pragma unroll
    for (int j = 0; j < RPW; j++) sum[j] = wave_sum(sum[j]);
#pragma unroll
    for (int j = 0; j < RPW; j++) {
      float *srow = lds + (wave + ATT_WAVES * j) * p.pitch;
      const float inv = 1.0f / sum[j];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int c = 4 * lane + 256 * i;
        if (c < ncols) {
          f32x4 t;
#pragma unroll
          for (int e = 0; e < 4; e++) t[e] = v[j][i][e] * inv;
          *reinterpret_cast<f32x4 *>(srow + c) = t;
        }
      }
    }
  }
  __syncthreads();

  // ---- 3. output: this wavefront's key blocks -----------------------------------------
  f32x16 o[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
    o[nb] = f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if constexpr (NB == 1) {
#pragma unroll
    for (int it = 0; it < PER_WAVE; it++) {
      const int kc = wave + ATT_WAVES * it;
      if (kc >= ncb) break;
      const float *prow = lds + li * p.pitch + kc * 32 + 16 * half;
      f32x4 pa[4];
#pragma unroll
      for (int c = 0; c < 4; c++) pa[c] = *reinterpret_cast<const f32x4 *>(prow + 4 * c);
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int s = 0; s < 16; s++)
          o[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[s >> 2][s & 3], vb[it][nb][s], o[nb], 0, 0, 0);
    }
  } else {
    for (int kc = wave; kc < ncb; kc += ATT_WAVES) {
      const int key0 = kc * 32 + 16 * half;
      const float *prow = lds + li * p.pitch + key0;
      f32x4 pa[4];
#pragma unroll
      for (int c = 0; c < 4; c++) pa[c] = *reinterpret_cast<const f32x4 *>(prow + 4 * c);
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        float vn[16];
#pragma unroll
        for (int s = 0; s < 16; s++) {
          const int key = key0 + s;
          const float t = V[(long long)(key < p.tk ? key : p.tk - 1) * p.sVj + nb * 32 + li];
          vn[s] = key < p.tk ? t : 0.0f;
        }
#pragma unroll
        for (int s = 0; s < 16; s++)
          o[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[s >> 2][s & 3], vn[s], o[nb], 0, 0, 0);
      }
    }
  }
  __syncthreads();  // every wavefront has read its part of P: the block is free

  // ---- partial blocks added in wavefront order ----------------------------------------
  constexpr int OP = HD + 1;  // row pitch of a partial block
  {
    float *mine = lds + wave * (ATT_ROWS * OP);
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int row = 8 * (r >> 2) + 4 * half + (r & 3);
        mine[row * OP + nb * 32 + li] = o[nb][r];
      }
  }
  __syncthreads();
  float *Y = p.Y + (long long)b * p.sYb;
  for (int cell = tid; cell < ATT_ROWS * HD; cell += 64 * ATT_WAVES) {
    const int row = cell / HD, col = cell - row * HD;
    float sum = lds[row * OP + col];
#pragma unroll
    for (int w = 1; w < ATT_WAVES; w++) sum += lds[w * (ATT_ROWS * OP) + row * OP + col];
    if (row0 + row < p.tq) Y[(long long)(row0 + row) * p.sYi + col] = sum;
  }
}

int lds_pitch(int tk) {
  int pitch = (tk + 31) / 32 * 32;
  if ((pitch / 4) % 2 == 0) pitch += 4;  // rows 16 bytes apart modulo the banks: no conflicts in step 3
  return pitch;
}

template <int HD, int ATT_WAVES>
int launch_attention(const AttParams &p, int batch) {
  // the scores block, and later the wavefronts' partial outputs, whichever is larger
  size_t bytes = (size_t)ATT_ROWS * p.pitch * 4;
  const size_t partials = (size_t)ATT_WAVES * ATT_ROWS * (HD + 1) * 4;
  if (partials > bytes) bytes = partials;
  hipLaunchKernelGGL((attention_rows_kernel<HD, ATT_WAVES>), dim3((unsigned)((long long)batch * p.row_blocks)),
                     dim3(64 * ATT_WAVES), bytes, wdh::stream(), p);
  WDH_LAUNCH_CHECK();
  return WDH_OK;
}

}  // namespace

namespace wdh {
// More than 64 KB of dynamic LDS has to be asked for once per kernel and device (called by
// wdh_init with the device current, so that no launch -- captured ones included -- has to).
int init_attention() {
  const int limit = 160 * 1024;
  WDH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(attention_rows_kernel<32, 16>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, limit));
  WDH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(attention_rows_kernel<64, 8>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, limit));
  WDH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(attention_rows_kernel<128, 8>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, limit));
  return WDH_OK;
}
}  // namespace wdh

using wdh::fail;

extern "C" int wdh_attention(wdh_buf hQ, wdh_buf hK, wdh_buf hV, wdh_buf hY, int batch, int tq,
                             int tk, int d, int64_t sQb, int64_t sQi, int64_t sKb, int64_t sKj,
                             int64_t sVb, int64_t sVj, int64_t sYb, int64_t sYi, float alpha) {
  WDH_REQUIRE_INIT();
  WDH_REQUIRE_COMPUTE_LANE();
  if (batch < 0 || tq < 0 || tk < 0 || d < 0) return fail(WDH_EINVAL, "wdh_attention: negative extent");
  if (d != 32 && d != 64 && d != 128)
    return fail(WDH_EINVAL, "wdh_attention: head dimension %d (32, 64 and 128 are built)", d);
  if (tk > ATT_MAX_KEYS)
    return fail(WDH_EINVAL, "wdh_attention: %d keys (at most %d: a block of scores has to fit in LDS)", tk,
                ATT_MAX_KEYS);
  if (sQb < 0 || sQi < 0 || sKb < 0 || sKj < 0 || sVb < 0 || sVj < 0 || sYb < 0 || sYi < 0)
    return fail(WDH_EINVAL, "wdh_attention: negative stride");
  if (batch == 0 || tq == 0) return WDH_OK;
  if (tk == 0) return fail(WDH_EINVAL, "wdh_attention: no keys");
  if ((sQb | sQi | sKb | sKj) % 4 != 0)
    return fail(WDH_EINVAL, "wdh_attention: strides of Q and K must be multiples of 4 elements");
  const long long row_blocks = (tq + ATT_ROWS - 1) / ATT_ROWS;
  if (batch * row_blocks > 0x7fffffffLL) return fail(WDH_EINVAL, "wdh_attention: too many row blocks");
  auto span = [](long long n0, long long s0, long long n1, long long s1, long long inner) {
    return (n0 - 1) * s0 + (n1 - 1) * s1 + inner;
  };
  void *pq, *pk, *pv, *py;
  if (!wdh::operand(hQ, (size_t)span(batch, sQb, tq, sQi, d) * 4, "wdh_attention: Q", &pq)) return WDH_EINVAL;
  if (!wdh::operand(hK, (size_t)span(batch, sKb, tk, sKj, d) * 4, "wdh_attention: K", &pk)) return WDH_EINVAL;
  if (!wdh::operand(hV, (size_t)span(batch, sVb, tk, sVj, d) * 4, "wdh_attention: V", &pv)) return WDH_EINVAL;
  if (!wdh::operand(hY, (size_t)span(batch, sYb, tq, sYi, d) * 4, "wdh_attention: Y", &py)) return WDH_EINVAL;
  if ((((uintptr_t)pq | (uintptr_t)pk) & 15) != 0)
    return fail(WDH_EINVAL, "wdh_attention: Q and K must be 16-byte aligned");
  if (py == pq || py == pk || py == pv) return fail(WDH_EINVAL, "wdh_attention: Y aliases an input");
  AttParams p;
  p.Q = (const float *)pq; p.K = (const float *)pk; p.V = (const float *)pv; p.Y = (float *)py;
  p.tq = tq; p.tk = tk; p.pitch = lds_pitch(tk); p.row_blocks = (int)row_blocks;
  p.sQb = sQb; p.sQi = sQi; p.sKb = sKb; p.sKj = sKj; p.sVb = sVb; p.sVj = sVj; p.sYb = sYb; p.sYi = sYi;
  p.alpha = alpha;
  if (d == 32) return launch_attention<32, 16>(p, batch);
  if (d == 64) return launch_attention<64, 8>(p, batch);
  return launch_attention<128, 8>(p, batch);
}
