// What an attention without rotation does to a step's projected rows before the scores: every head of q and
// k is divided by its root mean square (an RMS norm without a gain: x / sqrt(mean(x^2) + eps)), q is
// multiplied by a temperature that grows with the logarithm of the position,
//     1 + coef * log(1 + (p + 1) div every)        (div: integer division),
// and k and v go to their pages.  Values may have a head size of their own.  Rows are [q: nh*hd | k: nkv*hd |
// v: nkv*vd]; q and k are changed in place (the attention kernel reads q from the row).  Sums, roots and
// the temperature are float32.  Heads may be stored wider than they are (zeros behind their norm_dim channels, so
// that keys and values have one size that the matrix-core kernels take): the mean of the squares is over norm_dim.
#include "common.h"

namespace {
template <typename T>
__global__ __launch_bounds__(64) void qk_unit_kv_kernel(T* __restrict__ rows, long ld, T* __restrict__ kpages, T* __restrict__ vpages,
                                                        const int* __restrict__ pos, const int* __restrict__ row_req,
                                                        const int* __restrict__ table, int max_pages, int page_size, int num_pages,
                                                        int nh, int nkv, int hd, int vd, float eps, int unit, int norm_dim,
                                                        float temp_coef, int temp_every) {
  const int n = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int p = pos[n];
  T* row = rows + (size_t)n * ld;
  T* x = row + (size_t)head * hd;   // q heads first, then k heads: both of size hd
  float ss = 0.f;
  if (unit)
    for (int e = lane; e < hd; e += WAVE) {
      const float v = to_float(x[e]);
      ss = fmaf(v, v, ss);
    }
  float scale = unit ? 1.0f / sqrtf(wave_sum(ss) / (float)norm_dim + eps) : 1.0f;
  if (head < nh) {
    if (temp_every > 0) scale *= 1.0f + temp_coef * logf((float)((p + 1) / temp_every) + 1.0f);
    for (int e = lane; e < hd; e += WAVE) x[e] = from_float<T>(to_float(x[e]) * scale);
    return;
  }
  const int g = head - nh;
  int page = kpages ? table[(size_t)row_req[n] * max_pages + p / page_size] : 0;
  page = page < 0 ? 0 : (page >= num_pages ? num_pages - 1 : page);   // never write outside the pool
  const size_t at = ((size_t)page * nkv + g) * page_size + p % page_size;
  for (int e = lane; e < hd; e += WAVE) {
    const T v = from_float<T>(to_float(x[e]) * scale);
    x[e] = v;
    if (kpages) kpages[at * hd + e] = v;
  }
  if (vpages) {
    const T* v = row + (size_t)(nh + nkv) * hd + (size_t)g * vd;
    for (int e = lane; e < vd; e += WAVE) vpages[at * vd + e] = v[e];
  }
}
}  // namespace

GIBBS_EXPORT int gibbs_qk_unit_kv(void* rows, long ld, void* kpages, void* vpages, int dtype, const int* pos, const int* row_req,
                                  const int* table, int max_pages, int page_size, int num_pages, int n_rows, int nh, int nkv,
                                  int hd, int vd, float eps, int unit, int norm_dim, float temp_coef, int temp_every,
                                  hipStream_t stream) {
  if (norm_dim <= 0) norm_dim = hd;
  GIBBS_REQUIRE(rows && pos && n_rows > 0 && nh > 0 && nkv >= 0 && hd > 0 && vd > 0, "qk_unit_kv: bad operands rows=%d heads=%d kv=%d", n_rows, nh, nkv);
  GIBBS_REQUIRE(ld >= (long)(nh + nkv) * hd + (long)nkv * vd, "qk_unit_kv: rows of %ld values cannot hold q, k and v", ld);
  GIBBS_REQUIRE(!kpages || (vpages && row_req && table && max_pages > 0 && page_size > 0 && num_pages > 0), "qk_unit_kv: pages without their table");
  const dim3 grid(n_rows, nh + nkv);
  if (dtype == GIBBS_F32)
    qk_unit_kv_kernel<float><<<grid, 64, 0, stream>>>((float*)rows, ld, (float*)kpages, (float*)vpages, pos, row_req, table, max_pages,
                                                      page_size, num_pages, nh, nkv, hd, vd, eps, unit, norm_dim, temp_coef, temp_every);
  else if (dtype == GIBBS_BF16)
    qk_unit_kv_kernel<bf16><<<grid, 64, 0, stream>>>((bf16*)rows, ld, (bf16*)kpages, (bf16*)vpages, pos, row_req, table, max_pages,
                                                     page_size, num_pages, nh, nkv, hd, vd, eps, unit, norm_dim, temp_coef, temp_every);
  else
    return gibbs_fail("qk_unit_kv: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("qk_unit_kv");
}
