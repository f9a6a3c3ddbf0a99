// Paged causal grouped-query attention, one workgroup per (token row, q head),
// for any head size that is a multiple of 16 up to 256, any number of heads and
// groups, any page size, with an optional window.  This is the attention of the
// float32 path (chunk rows and decode rows alike) and the fallback of the
// bfloat16 path for head sizes its fast kernels refuse.
//
// A workgroup is 16 groups of 16 lanes.  Lane j of a group owns dims j, j+16, ...
// Group g walks keys lo+g, lo+g+16, ... with an online softmax; the 16 partial
// results are merged in LDS with the usual rescaling.  Scores, softmax statistics
// and the output accumulate in 32-bit.
#include "common.h"
#include "tinyinfer_kernels.h"

TI_ERROR_API

#define AG_GROUPS 16
#define AG_LANES 16

template <typename T, int DPL>
__global__ void __launch_bounds__(256)
attention_rows_kernel(const T* __restrict__ q, const T* __restrict__ pool, const int* __restrict__ table,
                      int table_stride, const int* __restrict__ pos, const int* __restrict__ slot,
                      T* __restrict__ out, int n_head, int n_kv, int P, float scale, int window) {
  constexpr int HD = DPL * AG_LANES;
  __shared__ float s_o[AG_GROUPS][HD];
  __shared__ float s_m[AG_GROUPS], s_l[AG_GROUPS];
  const int m = blockIdx.x, h = blockIdx.y;
  const int g = threadIdx.x / AG_LANES, lane = threadIdx.x % AG_LANES;
  const int kvh = h / (n_head / n_kv);
  const int p_q = pos[m];
  const int lo = (window > 0 && p_q - window + 1 > 0) ? p_q - window + 1 : 0;
  const int* tab = table + (size_t)slot[m] * table_stride;
  const size_t page_elems = (size_t)2 * n_kv * P * HD;
  const size_t k_off = (size_t)kvh * P * HD;
  const size_t v_off = ((size_t)n_kv + kvh) * P * HD;

  float qv[DPL], o[DPL];
  const T* qh = q + ((size_t)m * n_head + h) * HD;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    qv[i] = ld<T>(qh + lane + i * AG_LANES) * scale;
    o[i] = 0.f;
  }
  float mx = -INFINITY, l = 0.f;
  for (int p = lo + g; p <= p_q; p += AG_GROUPS) {
    const int page = tab[p / P];
    if (page < 0) continue;   // never happens for a reserved request; never read astray
    const T* kp = pool + (size_t)page * page_elems + k_off + (size_t)(p % P) * HD;
    const T* vp = pool + (size_t)page * page_elems + v_off + (p % P);   // values lie transposed: [d][row]
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) s = fmaf(qv[i], ld<T>(kp + lane + i * AG_LANES), s);
    s = group_sum<AG_LANES>(s);
    const float m_new = fmaxf(mx, s);
    const float alpha = expf(mx - m_new);   // exp(-inf) = 0 on the first key
    const float w = expf(s - m_new);
    l = l * alpha + w;
#pragma unroll
    for (int i = 0; i < DPL; ++i) o[i] = o[i] * alpha + w * ld<T>(vp + (size_t)(lane + i * AG_LANES) * P);
    mx = m_new;
  }
#pragma unroll
  for (int i = 0; i < DPL; ++i) s_o[g][lane + i * AG_LANES] = o[i];
  if (lane == 0) {
    s_m[g] = mx;
    s_l[g] = l;
  }
  __syncthreads();
  // merge: every thread takes dims tid, tid+256, ... (HD <= 256: at most one)
  for (int d = threadIdx.x; d < HD; d += 256) {
    float mm = -INFINITY;
#pragma unroll
    for (int j = 0; j < AG_GROUPS; ++j) mm = fmaxf(mm, s_m[j]);
    float lt = 0.f, acc = 0.f;
#pragma unroll
    for (int j = 0; j < AG_GROUPS; ++j) {
      const float w = (s_m[j] == -INFINITY) ? 0.f : expf(s_m[j] - mm);
      lt += s_l[j] * w;
      acc += s_o[j][d] * w;
    }
    st<T>(out + ((size_t)m * n_head + h) * HD + d, acc / lt);
  }
}

template <typename T>
static int launch_rows(int dpl, dim3 grid, const void* q, const void* pool, const int* table, int table_stride,
                       const int* pos, const int* slot, void* out, int n_head, int n_kv, int P, float scale,
                       int window, hipStream_t stream) {
#define AG_CASE(D)                                                                                     \
  case D:                                                                                              \
    attention_rows_kernel<T, D><<<grid, 256, 0, stream>>>((const T*)q, (const T*)pool, table,           \
                                                          table_stride, pos, slot, (T*)out, n_head,    \
                                                          n_kv, P, scale, window);                     \
    break;
  switch (dpl) {
    AG_CASE(1) AG_CASE(2) AG_CASE(3) AG_CASE(4) AG_CASE(5) AG_CASE(6) AG_CASE(7) AG_CASE(8)
    AG_CASE(9) AG_CASE(10) AG_CASE(11) AG_CASE(12) AG_CASE(13) AG_CASE(14) AG_CASE(15) AG_CASE(16)
    default:
      return 1;
  }
#undef AG_CASE
  return 0;
}

// q, out: [M, n_head, hd] in T; pool: [pages][K: [n_kv][P][hd] | V: [n_kv][hd][P]] in T;
// table: [slots][table_stride];
// pos, slot: [M].  window <= 0: all keys up to the row's own position.
extern "C" int ti_attention_rows(int dtype, const void* q, const void* pool, const int* table, int table_stride,
                                 const int* pos, const int* slot, void* out, int M, int n_head, int n_kv,
                                 int hd, int page_size, float scale, int window, hipStream_t stream) {
  TI_REQUIRE(hd >= 16 && hd <= 256 && hd % 16 == 0,
             "attention: head_dim %d is not served (multiples of 16 up to 256)", hd);
  TI_REQUIRE(n_head > 0 && n_kv > 0 && n_head % n_kv == 0, "attention: heads %d / kv_heads %d", n_head, n_kv);
  TI_REQUIRE(n_head <= 65535, "attention: too many heads (%d)", n_head);
  TI_REQUIRE(page_size > 0 && table_stride > 0, "attention: bad page_size %d / table_stride %d", page_size, table_stride);
  if (M == 0) return 0;
  dim3 grid(M, n_head);
  int rc;
  if (dtype == TI_F32)
    rc = launch_rows<float>(hd / 16, grid, q, pool, table, table_stride, pos, slot, out, n_head, n_kv, page_size, scale, window, stream);
  else if (dtype == TI_BF16)
    rc = launch_rows<bf16_t>(hd / 16, grid, q, pool, table, table_stride, pos, slot, out, n_head, n_kv, page_size, scale, window, stream);
  else
    TI_REQUIRE(false, "attention: unknown dtype %d", dtype);
  TI_REQUIRE(rc == 0, "attention: no kernel for head_dim %d", hd);
  TI_LAUNCH_CHECK();
  return 0;
}
