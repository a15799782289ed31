// Kernels of the latent-attention mixer and of its neighbours in a model: an embedding that adds rows of a
// hashed token-pair table and of a learned position table, several residual streams that a layer reads as
// one weighted sum and writes through a small mixing matrix (hyper-connections), layer norm, the rotation
// of a latent attention's shared key part, per-head products with an output gate, and the polynomial-norm activation.
//
// Sums, norms, angles and the streams themselves are float32 whatever the run's activation type is.
#include "common.h"
#include <algorithm>

namespace {
// Elements a thread takes at a time: four floats (or bfloat16 values) where rows allow it, else one.
template <int V> struct FloatVec { float v[V]; };
template <int V> __device__ __forceinline__ FloatVec<V> load_vec(const float* p) {
  FloatVec<V> r;
  if constexpr (V == 4) { const float4 t = *(const float4*)p; r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w; }
  else r.v[0] = *p;
  return r;
}
template <int V> __device__ __forceinline__ FloatVec<V> load_vec(const bf16* p) {
  FloatVec<V> r;
  if constexpr (V == 4) {
    typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
    const bf16x4 t = *(const bf16x4*)p;
#pragma unroll
    for (int i = 0; i < 4; ++i) r.v[i] = (float)t[i];
  } else {
    r.v[0] = (float)*p;
  }
  return r;
}
template <int V> __device__ __forceinline__ void store_vec(float* p, const FloatVec<V>& r) {
  if constexpr (V == 4) *(float4*)p = float4{r.v[0], r.v[1], r.v[2], r.v[3]};
  else *p = r.v[0];
}
template <int V> __device__ __forceinline__ void store_vec(bf16* p, const FloatVec<V>& r) {
  if constexpr (V == 4) {
    typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
    *(bf16x4*)p = bf16x4{(bf16)r.v[0], (bf16)r.v[1], (bf16)r.v[2], (bf16)r.v[3]};
  } else {
    *p = (bf16)r.v[0];
  }
}

// Threads of a workgroup that owns a row of `per` vectors: few rows get wide workgroups (one pass over the row, every load in
// flight at once: such a step is a chain of short kernels that wait for memory), many rows get 256 threads.
int row_threads(int per, int n_rows) {
  if (n_rows <= 256 && per > 256) return std::min(1024, (per + 63) / 64 * 64);
  return per >= 512 ? 256 : (per >= 128 ? 128 : 64);
}

// ------------------------------------------------------------------------------------------------- embedding
// x[c][n][:] = table[id] + pair_table[row] + pos_table[pos], c = 0 .. copies - 1, with
//   row = buckets                                  for a sequence's first token (position 0)
//         (prev * mul_prev + id * mul_cur) mod buckets   otherwise,
// prev being the row before in this step, or, for the first row of a request's portion, the token that the
// request's state slot holds (what gibbs_store_last_token left there).
template <typename T, int V>
__global__ void embed_tables_kernel(const T* __restrict__ table, const T* __restrict__ pair_table, const T* __restrict__ pos_table,
                                    const int* __restrict__ ids, const int* __restrict__ pos, const int* __restrict__ row_req,
                                    const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ prev,
                                    long slot_stride, float* __restrict__ x, int copies, int n_rows, int hidden, int vocab,
                                    int buckets, int mul_prev, int mul_cur, int pos_len) {
  const int n = blockIdx.x;
  int id = ids[n];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);      // (never read outside the table)
  const T* row = table + (size_t)id * hidden;
  const T* pair = nullptr;
  const int p = pos[n];
  if (pair_table) {
    long r = buckets;
    if (p > 0) {
      const int req = row_req[n];
      int before = n > cu[req] ? ids[n - 1] : prev[(size_t)slot[req] * slot_stride];
      before = before < 0 ? 0 : (before >= vocab ? vocab - 1 : before);
      r = ((long)before * mul_prev + (long)id * mul_cur) % buckets;
    }
    pair = pair_table + (size_t)r * hidden;
  }
  const T* at = pos_table ? pos_table + (size_t)min(max(p, 0), pos_len - 1) * hidden : nullptr;
  for (int i = threadIdx.x * V; i < hidden; i += blockDim.x * V) {
    FloatVec<V> v = load_vec<V>(row + i);
    if (pair) {
      const FloatVec<V> more = load_vec<V>(pair + i);
#pragma unroll
      for (int e = 0; e < V; ++e) v.v[e] += more.v[e];
    }
    if (at) {
      const FloatVec<V> more = load_vec<V>(at + i);
#pragma unroll
      for (int e = 0; e < V; ++e) v.v[e] += more.v[e];
    }
    for (int c = 0; c < copies; ++c) store_vec<V>(x + ((size_t)c * n_rows + n) * hidden + i, v);
  }
}

__global__ void store_last_token_kernel(const int* __restrict__ ids, const int* __restrict__ cu, const int* __restrict__ slot,
                                        int* __restrict__ prev, long slot_stride, int n_req) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n_req || cu[r + 1] <= cu[r]) return;
  prev[(size_t)slot[r] * slot_stride] = ids[cu[r + 1] - 1];
}

// ------------------------------------------------------------------------------------------------- streams
// One workgroup per row.  WRITE: first all streams are written at once from the old ones,
//   x[t] <- sum_s mix[s][t] x[s] + out_coef[t] * y, s ascending, y the delta (one part in its type, or float32 partial
//   sums added in ascending order);
// then (coef_in, or NORM without WRITE) out[j][:] = norm(u), u = sum_s coef[s] x[s][row j][:] of the streams as they are
// now (coef null: every stream counts 1), s ascending.
//   kind 0: u / sqrt(mean(u^2) + eps) * gain;  kind 1: (u - mean) / sqrt(mean((u - mean)^2) + eps) * gain + bias.
// gain or bias null: 1 and 0.  u is kept in LDS (hidden floats).  The loads of all streams of an element are asked for
// together (S is a template parameter: the loop over the streams has no waits inside).
template <int S, int V, typename T, typename TD, bool WRITE, bool NORM>
__global__ void streams_kernel(float* __restrict__ x, long stream_stride, const float* __restrict__ mix,
                               const float* __restrict__ out_coef, const TD* __restrict__ delta, int parts, long part_stride,
                               const float* __restrict__ coef, int kind, const float* __restrict__ gain,
                               const float* __restrict__ bias, float eps, T* __restrict__ out, const int* __restrict__ rows,
                               int hidden) {
  extern __shared__ float u[];
  __shared__ float scratch[16];
  const int j = blockIdx.x;
  const size_t row = rows ? rows[j] : j;
  float m[S][S], oc[S], ci[S];
#pragma unroll
  for (int s = 0; s < S; ++s) {
    ci[s] = (NORM && coef) ? coef[s] : 1.f;
    if constexpr (WRITE) {
      oc[s] = out_coef[s];
#pragma unroll
      for (int t = 0; t < S; ++t) m[s][t] = mix[s * S + t];
    }
  }
  float sum = 0.f;
  for (int i = threadIdx.x * V; i < hidden; i += blockDim.x * V) {
    FloatVec<V> cur[S];
#pragma unroll
    for (int s = 0; s < S; ++s) cur[s] = load_vec<V>(x + (size_t)s * stream_stride + row * hidden + i);
    if constexpr (WRITE) {
      // (partial sums: four loads in flight at a time, added in ascending order)
      FloatVec<V> y = load_vec<V>(delta + row * hidden + i);
      for (int p = 1; p < parts; p += 4) {
        FloatVec<V> more[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) more[k] = load_vec<V>(delta + (size_t)min(p + k, parts - 1) * part_stride + row * hidden + i);
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (p + k < parts) {
#pragma unroll
            for (int e = 0; e < V; ++e) y.v[e] += more[k].v[e];
          }
      }
      FloatVec<V> fresh[S];
#pragma unroll
      for (int t = 0; t < S; ++t) {
#pragma unroll
        for (int e = 0; e < V; ++e) {
          float acc = 0.f;
#pragma unroll
          for (int s = 0; s < S; ++s) acc = fmaf(m[s][t], cur[s].v[e], acc);
          fresh[t].v[e] = fmaf(oc[t], y.v[e], acc);
        }
        store_vec<V>(x + (size_t)t * stream_stride + row * hidden + i, fresh[t]);
      }
#pragma unroll
      for (int t = 0; t < S; ++t) cur[t] = fresh[t];
    }
    if constexpr (NORM) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < S; ++s) v = coef ? fmaf(ci[s], cur[s].v[e], v) : v + cur[s].v[e];
        u[i + e] = v;
        sum += v;
      }
    }
  }
  if constexpr (!NORM) return;
  float mean = 0.f;
  if (kind == 1) mean = block_sum(sum, scratch) / (float)hidden;
  float sq = 0.f;
  for (int i = threadIdx.x * V; i < hidden; i += blockDim.x * V) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float d = u[i + e] - mean;
      sq = fmaf(d, d, sq);
    }
  }
  const float r = 1.0f / sqrtf(block_sum(sq, scratch) / (float)hidden + eps);
  for (int i = threadIdx.x * V; i < hidden; i += blockDim.x * V) {
    FloatVec<V> o;
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float v = (u[i + e] - mean) * r;
      if (gain) v *= gain[i + e];
      if (bias && kind == 1) v += bias[i + e];
      o.v[e] = v;
    }
    store_vec<V>(out + (size_t)j * hidden + i, o);
  }
}

// ------------------------------------------------------------------------------------------------- rows
// out[n][:] = in[n][:width] / sqrt(mean(in^2) + eps) * gain; one workgroup per row, V values a thread at a time.
template <typename T, int V>
__global__ void rms_rows_ld_kernel(const T* __restrict__ in, long ld_in, const float* __restrict__ gain, float eps,
                                   T* __restrict__ out, long ld_out, int width) {
  __shared__ float scratch[16];
  const T* src = in + (size_t)blockIdx.x * ld_in;
  float sq = 0.f;
#pragma unroll 4
  for (int i = threadIdx.x * V; i < width; i += blockDim.x * V) {
    const FloatVec<V> r = load_vec<V>(src + i);
#pragma unroll
    for (int e = 0; e < V; ++e) sq = fmaf(r.v[e], r.v[e], sq);
  }
  const float r = 1.0f / sqrtf(block_sum(sq, scratch) / (float)width + eps);
#pragma unroll 4
  for (int i = threadIdx.x * V; i < width; i += blockDim.x * V) {
    FloatVec<V> o = load_vec<V>(src + i);
#pragma unroll
    for (int e = 0; e < V; ++e) o.v[e] = o.v[e] * r * (gain ? gain[i + e] : 1.f);
    store_vec<V>(out + (size_t)blockIdx.x * ld_out + i, o);
  }
}

// The pair (u, v) at position p becomes (u cos a - v sin a, v cos a + u sin a), a = float(p) * inv_freq[i].
// variant 0: pairs (i, i + dims / 2); 1: pairs (2 i, 2 i + 1); entries from `dims` on pass unchanged.
template <typename T>
__device__ __forceinline__ void rotate_into(const T* __restrict__ src, T* __restrict__ dst, int width, int dims, int variant,
                                            const float* __restrict__ inv_freq, float p, int lane, int lanes) {
  const int half = dims / 2;
  for (int i = lane; i < half; i += lanes) {
    const int a = variant ? 2 * i : i, b = variant ? 2 * i + 1 : i + half;
    const float angle = p * inv_freq[i];
    const float c = cosf(angle), s = sinf(angle);
    const float u = to_float(src[a]), v = to_float(src[b]);
    dst[a] = from_float<T>(u * c - v * s);
    dst[b] = from_float<T>(v * c + u * s);
  }
  for (int i = dims + lane; i < width; i += lanes) dst[i] = src[i];
}

// What a latent attention does to a step's rows before the scores: per row n at position p of request r,
//   the cached row  page[p] = [ kv[n][:rank] / rms * gain | rotate(kv[n][rank : rank + rot]) ]   (one per token, shared by all heads)
//   the queries' rotated parts  q_out[n][h][rank : rank + rot] = rotate(q[n][h][dim : dim + rot]).
// (The queries' first `rank` entries, their unrotated parts taken through the keys' up-projection, are another kernel's.)
// One workgroup of 256 threads per row: its first wave makes the cached row, all threads share the heads' pairs.
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(const T* __restrict__ kv, long ld_kv, const T* __restrict__ q, long ld_q,
                                                             T* __restrict__ q_out, long ld_qo, T* __restrict__ pages,
                                                             const float* __restrict__ gain, float eps, const float* __restrict__ inv_freq,
                                                             int dims, int variant, const int* __restrict__ pos,
                                                             const int* __restrict__ row_req, const int* __restrict__ table, int max_pages,
                                                             int page_size, int num_pages, int nh, int dim, int rot, int rank) {
  const int n = blockIdx.x, lane = threadIdx.x % WAVE;
  const int p = pos[n];
  if (threadIdx.x < WAVE) {
    int page = table[(size_t)row_req[n] * max_pages + p / page_size];
    page = page < 0 ? 0 : (page >= num_pages ? num_pages - 1 : page);      // never write outside the pool
    T* dst = pages + ((size_t)page * page_size + p % page_size) * (rank + rot);
    const T* src = kv + (size_t)n * ld_kv;
    float sq = 0.f;
    for (int i = lane; i < rank; i += WAVE) {
      const float v = to_float(src[i]);
      sq = fmaf(v, v, sq);
    }
    const float r = 1.0f / sqrtf(wave_sum(sq) / (float)rank + eps);
    for (int i = lane; i < rank; i += WAVE) dst[i] = from_float<T>(to_float(src[i]) * r * (gain ? gain[i] : 1.f));
    rotate_into(src + rank, dst + rank, rot, dims, variant, inv_freq, (float)p, lane, WAVE);
  }
  // the heads' rotated parts: pair i of head h for every (h, i); what does not turn is copied
  const int half = dims / 2;
  const T* qs = q + (size_t)n * ld_q + dim;
  T* qd = q_out + (size_t)n * ld_qo + rank;
  for (int e = threadIdx.x; e < nh * half; e += blockDim.x) {
    const int h = e / half, i = e % half;
    const int a = variant ? 2 * i : i, b = variant ? 2 * i + 1 : i + half;
    const float angle = (float)p * inv_freq[i];
    const float c = cosf(angle), s = sinf(angle);
    const T* src = qs + (size_t)h * (dim + rot);
    T* dst = qd + (size_t)h * (rank + rot);
    const float u = to_float(src[a]), v = to_float(src[b]);
    dst[a] = from_float<T>(u * c - v * s);
    dst[b] = from_float<T>(v * c + u * s);
  }
  const int rest = rot - dims;
  for (int e = threadIdx.x; e < nh * rest; e += blockDim.x) {
    const int h = e / rest, i = dims + e % rest;
    q_out[(size_t)n * ld_qo + (size_t)h * (rank + rot) + rank + i] = q[(size_t)n * ld_q + (size_t)h * (dim + rot) + dim + i];
  }
}

// out = a N(z) + b N(z^2) + c N(z^3) + e over a row of F values, N(v) = v / sqrt(mean(v^2) + eps), powers element by element.
// One workgroup per row; the row is read once, V values a thread at a time, and kept between the sums and the result:
// KEEP 2 in registers (up to 8 vectors a thread, all loads in flight at once), KEEP 1 in LDS (F floats), KEEP 0 read again.
template <typename T, int V, int KEEP>
__global__ void poly_norm_kernel(const T* __restrict__ z, T* __restrict__ out, const float* __restrict__ coef, float eps, int F) {
  extern __shared__ float kept[];
  __shared__ float scratch[16];
  const T* src = z + (size_t)blockIdx.x * F;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  FloatVec<V> mine[KEEP == 2 ? 8 : 1];
  if constexpr (KEEP == 2) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = (threadIdx.x + j * blockDim.x) * V;
      if (i < F) mine[j] = load_vec<V>(src + i);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = (threadIdx.x + j * blockDim.x) * V;
      if (i >= F) continue;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float v = mine[j].v[e], v2 = v * v;
        s2 += v2;
        s4 = fmaf(v2, v2, s4);
        s6 = fmaf(v2 * v, v2 * v, s6);
      }
    }
  } else {
#pragma unroll 4
    for (int i = threadIdx.x * V; i < F; i += blockDim.x * V) {
      const FloatVec<V> r = load_vec<V>(src + i);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float v = r.v[e], v2 = v * v;
        if constexpr (KEEP == 1) kept[i + e] = v;
        s2 += v2;
        s4 = fmaf(v2, v2, s4);
        s6 = fmaf(v2 * v, v2 * v, s6);
      }
    }
  }
  const float r1 = coef[0] / sqrtf(block_sum(s2, scratch) / (float)F + eps);
  const float r2 = coef[1] / sqrtf(block_sum(s4, scratch) / (float)F + eps);
  const float r3 = coef[2] / sqrtf(block_sum(s6, scratch) / (float)F + eps);
  const float c0 = coef[3];
  auto result = [&](FloatVec<V> r) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      const float v = r.v[e], v2 = v * v;
      r.v[e] = fmaf(r1, v, fmaf(r2, v2, fmaf(r3, v2 * v, c0)));
    }
    return r;
  };
  if constexpr (KEEP == 2) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = (threadIdx.x + j * blockDim.x) * V;
      if (i < F) store_vec<V>(out + (size_t)blockIdx.x * F + i, result(mine[j]));
    }
  } else {
#pragma unroll 4
    for (int i = threadIdx.x * V; i < F; i += blockDim.x * V) {
      FloatVec<V> r;
      if constexpr (KEEP == 1) {
#pragma unroll
        for (int e = 0; e < V; ++e) r.v[e] = kept[i + e];
      } else {
        r = load_vec<V>(src + i);
      }
      store_vec<V>(out + (size_t)blockIdx.x * F + i, result(r));
    }
  }
}

// ------------------------------------------------------------------------------------------------- per-head products
// Y[n][h][o] = sum_k X[n][h][k] W[h][o][k] for every head h: a product per head over slices of the same rows
// (X + h * head_x, row stride ldx; W + h * head_w, row stride ldw; Y + h * head_y, row stride ldy).
// With G (row stride ldg, head_g apart per head) every result is multiplied by sigmoid(G[n][h][o]) before it is stored.
// Plain FMA, every element in ascending k: the 32-bit path, and bfloat16 slices that are not 16-byte aligned.
constexpr int TM = 64, TN = 64, TK = 16;
template <typename T>
__global__ __launch_bounds__(256) void gemm_heads_plain_kernel(const T* __restrict__ X, long ldx, long head_x, const T* __restrict__ W,
                                                               long head_w, long ldw, T* __restrict__ Y, long ldy, long head_y, int N,
                                                               int O, int I, const T* __restrict__ G, long ldg, long head_g) {
  __shared__ float sa[TK][TM + 4];
  __shared__ float sw[TK][TN + 4];
  const int h = blockIdx.z;
  X += (size_t)h * head_x;
  W += (size_t)h * head_w;
  Y += (size_t)h * head_y;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int row0 = blockIdx.y * TM, col0 = blockIdx.x * TN;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < I; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = threadIdx.x + i * 256;
      const int r = e / TK, k = e % TK;
      const int gr = row0 + r, gc = col0 + r, gk = k0 + k;
      sa[k][r] = (gr < N && gk < I) ? to_float(X[(size_t)gr * ldx + gk]) : 0.f;
      sw[k][r] = (gc < O && gk < I) ? to_float(W[(size_t)gc * ldw + gk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = sa[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = sw[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gr = row0 + ty * 4 + i;
    if (gr >= N) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gc = col0 + tx * 4 + j;
      if (gc >= O) continue;
      float v = acc[i][j];
      if (G) v /= 1.0f + expf(-to_float(G[(size_t)gr * ldg + (size_t)h * head_g + gc]));
      Y[(size_t)gr * ldy + gc] = from_float<T>(v);
    }
  }
}

// The same on the matrix cores, for bfloat16 slices whose rows start at multiples of 16 bytes and whose inner
// size is a multiple of 8: a wave takes 16 rows x 64 features, four 16 x 16 x 32 products per step of k, both
// operands straight from memory (X and W are contiguous along k, which is the operand layout: lane l holds
// the 8 values k = (l / 16) * 8 .. + 8 of row or feature l % 16); a workgroup is 4 waves on 64 rows.  W is the
// first operand (the tile is Y^T = W X^T), so a lane's four results are four neighbouring features of one row:
// with VEC they leave (and the gate arrives) as one 8-byte access.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
template <bool VEC>
__global__ __launch_bounds__(256) void gemm_heads_mfma_kernel(const bf16* __restrict__ X, long ldx, long head_x, const bf16* __restrict__ W,
                                                              long head_w, long ldw, bf16* __restrict__ Y, long ldy, long head_y, int N,
                                                              int O, int I, const bf16* __restrict__ G, long ldg, long head_g) {
  const int h = blockIdx.z;
  X += (size_t)h * head_x;
  W += (size_t)h * head_w;
  Y += (size_t)h * head_y;
  if (G) G += (size_t)h * head_g;
  const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
  const int lr = lane % 16, lg = lane / 16;
  const int row = blockIdx.y * 64 + wave * 16 + lr;
  const int col0 = blockIdx.x * 64;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  floatx4 acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16* xr = X + (size_t)min(row, N - 1) * ldx;
  for (int k0 = 0; k0 < I; k0 += 32) {
    const int k = k0 + lg * 8;
    const bf16x8 x8 = (row < N && k < I) ? *(const bf16x8*)(xr + k) : zero8;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int col = col0 + t * 16 + lr;
      const bf16x8 w8 = (col < O && k < I) ? *(const bf16x8*)(W + (size_t)col * ldw + k) : zero8;
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w8, x8, acc[t], 0, 0, 0);
    }
  }
  // element i of a lane's result: feature (lane / 16) * 4 + i of the tile's 16, row lane % 16 of the wave's 16
  if (row >= N) return;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int col = col0 + t * 16 + lg * 4;
    if (VEC && col + 4 <= O) {
      float v[4] = {acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
      if (G) {
        const bf16x4 g4 = *(const bf16x4*)(G + (size_t)row * ldg + col);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] /= 1.0f + __expf(-(float)g4[i]);
      }
      *(bf16x4*)(Y + (size_t)row * ldy + col) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
      continue;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (col + i >= O) continue;
      float v = acc[t][i];
      if (G) v /= 1.0f + __expf(-(float)G[(size_t)row * ldg + col + i]);
      Y[(size_t)row * ldy + col + i] = (bf16)v;
    }
  }
}
}  // namespace

GIBBS_EXPORT int gibbs_embed_tables(const void* table, const void* pair_table, const void* pos_table, int dtype, const int* ids,
                                    const int* pos, const int* row_req, const int* cu, const int* slot, const int* prev,
                                    long slot_stride, float* x, int copies, int n, int hidden, int vocab, int buckets, int mul_prev,
                                    int mul_cur, int pos_len, hipStream_t stream) {
  GIBBS_REQUIRE(n >= 0 && hidden > 0 && vocab > 0 && copies >= 1, "embed_tables: bad sizes n=%d hidden=%d vocab=%d copies=%d", n, hidden, vocab, copies);
  GIBBS_REQUIRE(table && ids && pos && x, "embed_tables: the table, ids, positions and rows are needed");
  GIBBS_REQUIRE(!pair_table || (buckets > 0 && row_req && cu && slot && prev), "embed_tables: the pair table needs its buckets, the batch's layout and the requests' last tokens");
  GIBBS_REQUIRE(!pos_table || pos_len > 0, "embed_tables: an empty position table");
  if (n == 0) return 0;
  const bool vec = hidden % 4 == 0 && ((uintptr_t)table % 16) == 0 && ((uintptr_t)pair_table % 16) == 0 && ((uintptr_t)pos_table % 16) == 0 &&
                   ((uintptr_t)x % 16) == 0;
  const int threads = row_threads(vec ? hidden / 4 : hidden, n);
#define GIBBS_EMBED(T, V)                                                                                                        \
  embed_tables_kernel<T, V><<<n, threads, 0, stream>>>((const T*)table, (const T*)pair_table, (const T*)pos_table, ids, pos, row_req, cu, \
                                                       slot, prev, slot_stride, x, copies, n, hidden, vocab, buckets, mul_prev, mul_cur, pos_len)
  if (dtype == GIBBS_F32) {
    if (vec) GIBBS_EMBED(float, 4); else GIBBS_EMBED(float, 1);
  } else if (dtype == GIBBS_BF16) {
    if (vec) GIBBS_EMBED(bf16, 4); else GIBBS_EMBED(bf16, 1);
  } else {
    return gibbs_fail("embed_tables: unknown dtype %d", dtype);
  }
#undef GIBBS_EMBED
  GIBBS_LAUNCH_STATUS("embed_tables");
}

// prev[slot[r] * slot_stride] = the last token of request r's rows in this step (after the embedding has read what was there).
GIBBS_EXPORT int gibbs_store_last_token(const int* ids, const int* cu, const int* slot, int* prev, long slot_stride, int n_req,
                                        hipStream_t stream) {
  GIBBS_REQUIRE(n_req >= 0 && ids && cu && slot && prev, "store_last_token: missing operands");
  if (n_req == 0) return 0;
  store_last_token_kernel<<<ceil_div(n_req, 64), 64, 0, stream>>>(ids, cu, slot, prev, slot_stride, n_req);
  GIBBS_LAUNCH_STATUS("store_last_token");
}

namespace {
template <int S, int V, typename T, typename TD, bool WRITE, bool NORM>
void launch_streams_one(int n_rows, int hidden, hipStream_t stream, float* x, long stream_stride, const float* mix, const float* out_coef,
                        const TD* delta, int parts, long part_stride, const float* coef, int kind, const float* gain, const float* bias,
                        float eps, T* out, const int* rows) {
  const int threads = row_threads(hidden / V, n_rows);
  streams_kernel<S, V, T, TD, WRITE, NORM><<<n_rows, threads, NORM ? (size_t)hidden * 4 : 0, stream>>>(
      x, stream_stride, mix, out_coef, delta, parts, part_stride, coef, kind, gain, bias, eps, out, rows, hidden);
}
template <typename T, typename TD, bool WRITE, bool NORM>
int launch_streams(int streams, int n_rows, int hidden, hipStream_t stream, float* x, long stream_stride, const float* mix,
                   const float* out_coef, const TD* delta, int parts, long part_stride, const float* coef, int kind, const float* gain,
                   const float* bias, float eps, T* out, const int* rows) {
  const bool vec = hidden % 4 == 0 && stream_stride % 4 == 0 && part_stride % 4 == 0 && ((uintptr_t)x % 16) == 0 &&
                   ((uintptr_t)delta % 16) == 0 && ((uintptr_t)out % 16) == 0;
  switch (streams) {
#define GIBBS_STREAMS(S)                                                                                                          \
  case S:                                                                                                                         \
    if (vec) launch_streams_one<S, 4, T, TD, WRITE, NORM>(n_rows, hidden, stream, x, stream_stride, mix, out_coef, delta, parts,  \
                                                           part_stride, coef, kind, gain, bias, eps, out, rows);                  \
    else launch_streams_one<S, 1, T, TD, WRITE, NORM>(n_rows, hidden, stream, x, stream_stride, mix, out_coef, delta, parts,      \
                                                      part_stride, coef, kind, gain, bias, eps, out, rows);                       \
    break;
    GIBBS_STREAMS(1) GIBBS_STREAMS(2) GIBBS_STREAMS(3) GIBBS_STREAMS(4) GIBBS_STREAMS(5) GIBBS_STREAMS(6) GIBBS_STREAMS(7) GIBBS_STREAMS(8)
#undef GIBBS_STREAMS
    default: return gibbs_fail("streams: %d residual streams (1 to 8)", streams);
  }
  GIBBS_LAUNCH_STATUS("streams");
}
}  // namespace

// out [n_out, hidden] = norm(sum_s coef[s] x[s][row]) of all rows (rows null) or of `rows`; x [streams][.][hidden] float32.
GIBBS_EXPORT int gibbs_streams_norm(const float* x, int streams, long stream_stride, const float* coef, int kind, const float* gain,
                                    const float* bias, float eps, void* out, int dtype, const int* rows, int n_out, int hidden,
                                    hipStream_t stream) {
  GIBBS_REQUIRE(n_out >= 0 && hidden > 0 && streams >= 1 && (kind == 0 || kind == 1), "streams_norm: bad sizes rows=%d hidden=%d streams=%d kind=%d", n_out, hidden, streams, kind);
  GIBBS_REQUIRE(hidden <= 16000, "streams_norm: rows of %d values do not fit the workgroup's memory", hidden);
  if (n_out == 0) return 0;
  if (dtype == GIBBS_F32)
    return launch_streams<float, float, false, true>(streams, n_out, hidden, stream, (float*)x, stream_stride, nullptr, nullptr, nullptr, 0,
                                                     0, coef, kind, gain, bias, eps, (float*)out, rows);
  if (dtype == GIBBS_BF16)
    return launch_streams<bf16, float, false, true>(streams, n_out, hidden, stream, (float*)x, stream_stride, nullptr, nullptr, nullptr, 0,
                                                    0, coef, kind, gain, bias, eps, (bf16*)out, rows);
  return gibbs_fail("streams_norm: unknown dtype %d", dtype);
}

// x[t] <- sum_s mix[s][t] x[s] + out_coef[t] * delta for the n_rows rows of all streams at once, and, with `out`, the norm of
// the new streams' weighted sum (as gibbs_streams_norm, of all rows) in the same pass.  delta: [n_rows, hidden] in
// delta_dtype (parts 1), or float32 partial sums [parts][n_rows, hidden] (part_stride apart).
GIBBS_EXPORT int gibbs_streams_write_norm(float* x, int streams, long stream_stride, const float* mix, const float* out_coef,
                                          const void* delta, int delta_dtype, int parts, long part_stride, int n_rows, int hidden,
                                          const float* coef, int kind, const float* gain, const float* bias, float eps, void* out,
                                          int dtype, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && hidden > 0 && parts >= 1 && x && mix && out_coef && delta, "streams_write: missing operands");
  GIBBS_REQUIRE(parts == 1 || delta_dtype == GIBBS_F32, "streams_write: partial sums are float32");
  GIBBS_REQUIRE(!out || (hidden <= 16000 && (kind == 0 || kind == 1)), "streams_write: rows of %d values do not fit the workgroup's memory", hidden);
  if (n_rows == 0) return 0;
#define GIBBS_WRITE(T, TD)                                                                                                         \
  return out ? launch_streams<T, TD, true, true>(streams, n_rows, hidden, stream, x, stream_stride, mix, out_coef, (const TD*)delta, \
                                                 parts, part_stride, coef, kind, gain, bias, eps, (T*)out, nullptr)                \
             : launch_streams<T, TD, true, false>(streams, n_rows, hidden, stream, x, stream_stride, mix, out_coef, (const TD*)delta, \
                                                  parts, part_stride, nullptr, 0, nullptr, nullptr, 0.f, (T*)nullptr, nullptr)
  const bool out_bf16 = out && dtype == GIBBS_BF16;
  GIBBS_REQUIRE(!out || dtype == GIBBS_F32 || dtype == GIBBS_BF16, "streams_write: unknown dtype %d", dtype);
  if (delta_dtype == GIBBS_F32) {
    if (out_bf16) { GIBBS_WRITE(bf16, float); }
    GIBBS_WRITE(float, float);
  }
  if (delta_dtype == GIBBS_BF16) {
    if (out_bf16) { GIBBS_WRITE(bf16, bf16); }
    GIBBS_WRITE(float, bf16);
  }
#undef GIBBS_WRITE
  return gibbs_fail("streams_write: unknown dtype %d", delta_dtype);
}
// delta: [count] in delta_dtype (parts 1), or float32 partial sums [parts, count] (part_stride apart); the streams as one row.
GIBBS_EXPORT int gibbs_streams_write(float* x, int streams, long stream_stride, const float* mix, const float* out_coef,
                                     const void* delta, int delta_dtype, int parts, long part_stride, long count, hipStream_t stream) {
  GIBBS_REQUIRE(count >= 0, "streams_write: bad count");
  // (rows of 4,096 elements, the last one shorter: a workgroup per row)
  const int width = count % 4096 == 0 ? 4096 : (count % 1024 == 0 ? 1024 : 0);
  if (width) return gibbs_streams_write_norm(x, streams, stream_stride, mix, out_coef, delta, delta_dtype, parts, part_stride,
                                             (int)(count / width), width, nullptr, 0, nullptr, nullptr, 0.f, nullptr, 0, stream);
  return gibbs_streams_write_norm(x, streams, stream_stride, mix, out_coef, delta, delta_dtype, parts, part_stride, 1, (int)count, nullptr,
                                  0, nullptr, nullptr, 0.f, nullptr, 0, stream);
}

GIBBS_EXPORT int gibbs_rms_rows_ld(const void* in, long ld_in, const float* gain, float eps, void* out, long ld_out, int dtype, int n,
                                   int width, hipStream_t stream) {
  GIBBS_REQUIRE(n >= 0 && width > 0 && ld_in >= width && ld_out >= width, "rms_rows: bad sizes n=%d width=%d", n, width);
  GIBBS_REQUIRE(dtype == GIBBS_F32 || dtype == GIBBS_BF16, "rms_rows: unknown dtype %d", dtype);
  if (n == 0) return 0;
  const bool vec = width % 4 == 0 && ld_in % 4 == 0 && ld_out % 4 == 0 && ((uintptr_t)in % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int threads = row_threads(vec ? width / 4 : width, n);
  if (dtype == GIBBS_F32) {
    if (vec) rms_rows_ld_kernel<float, 4><<<n, threads, 0, stream>>>((const float*)in, ld_in, gain, eps, (float*)out, ld_out, width);
    else rms_rows_ld_kernel<float, 1><<<n, threads, 0, stream>>>((const float*)in, ld_in, gain, eps, (float*)out, ld_out, width);
  } else {
    if (vec) rms_rows_ld_kernel<bf16, 4><<<n, threads, 0, stream>>>((const bf16*)in, ld_in, gain, eps, (bf16*)out, ld_out, width);
    else rms_rows_ld_kernel<bf16, 1><<<n, threads, 0, stream>>>((const bf16*)in, ld_in, gain, eps, (bf16*)out, ld_out, width);
  }
  GIBBS_LAUNCH_STATUS("rms_rows");
}

// kv: rows [n, >= rank + rot] (the down-projection's result); q: rows of nh heads of dim + rot; q_out: rows of nh heads of
// rank + rot, of which this call fills the last rot; pages: [num_pages, page_size, rank + rot] of one layer.
GIBBS_EXPORT int gibbs_latent_prepare(const void* kv, long ld_kv, const void* q, long ld_q, void* q_out, long ld_qo, void* pages,
                                      int dtype, const float* gain, float eps, const float* inv_freq, int rot_dims, int variant,
                                      const int* pos, const int* row_req, const int* table, int max_pages, int page_size,
                                      int num_pages, int n_rows, int nh, int dim, int rot, int rank, hipStream_t stream) {
  GIBBS_REQUIRE(n_rows >= 0 && nh > 0 && dim >= 0 && rot >= 0 && rank > 0, "latent_prepare: bad sizes rows=%d heads=%d dim=%d rot=%d rank=%d", n_rows, nh, dim, rot, rank);
  GIBBS_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0 && (rot_dims == 0 || inv_freq), "latent_prepare: %d rotated dimensions of %d", rot_dims, rot);
  GIBBS_REQUIRE(variant == 0 || variant == 1, "latent_prepare: unknown pairing %d", variant);
  GIBBS_REQUIRE(ld_kv >= rank + rot && ld_q >= (long)nh * (dim + rot) && ld_qo >= (long)nh * (rank + rot), "latent_prepare: row strides shorter than rows");
  GIBBS_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0, "latent_prepare: bad cache geometry");
  if (n_rows == 0) return 0;
  const dim3 grid(n_rows);
  if (dtype == GIBBS_F32)
    latent_prepare_kernel<float><<<grid, 256, 0, stream>>>((const float*)kv, ld_kv, (const float*)q, ld_q, (float*)q_out, ld_qo, (float*)pages,
                                                            gain, eps, inv_freq, rot_dims, variant, pos, row_req, table, max_pages, page_size,
                                                            num_pages, nh, dim, rot, rank);
  else if (dtype == GIBBS_BF16)
    latent_prepare_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)kv, ld_kv, (const bf16*)q, ld_q, (bf16*)q_out, ld_qo, (bf16*)pages,
                                                           gain, eps, inv_freq, rot_dims, variant, pos, row_req, table, max_pages, page_size,
                                                           num_pages, nh, dim, rot, rank);
  else
    return gibbs_fail("latent_prepare: unknown dtype %d", dtype);
  GIBBS_LAUNCH_STATUS("latent_prepare");
}

// coef: float32 [4] on the device: a, b, c, e.
GIBBS_EXPORT int gibbs_poly_norm(const void* z, void* out, int dtype, const float* coef, float eps, int n, int F, hipStream_t stream) {
  GIBBS_REQUIRE(n >= 0 && F > 0 && coef, "poly_norm: bad sizes n=%d F=%d", n, F);
  GIBBS_REQUIRE(dtype == GIBBS_F32 || dtype == GIBBS_BF16, "poly_norm: unknown dtype %d", dtype);
  if (n == 0) return 0;
  const bool vec = F % 4 == 0 && ((uintptr_t)z % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int per = vec ? F / 4 : F;
  const int threads = row_threads(per, n);
  const int keep = per <= 8 * threads ? 2 : (F <= 16000 ? 1 : 0);
  const size_t lds = keep == 1 ? (size_t)F * 4 : 0;
#define GIBBS_POLY(T, V)                                                                                            \
  do {                                                                                                              \
    if (keep == 2) poly_norm_kernel<T, V, 2><<<n, threads, lds, stream>>>((const T*)z, (T*)out, coef, eps, F);      \
    else if (keep == 1) poly_norm_kernel<T, V, 1><<<n, threads, lds, stream>>>((const T*)z, (T*)out, coef, eps, F); \
    else poly_norm_kernel<T, V, 0><<<n, threads, lds, stream>>>((const T*)z, (T*)out, coef, eps, F);                \
  } while (0)
  if (dtype == GIBBS_F32) {
    if (vec) GIBBS_POLY(float, 4); else GIBBS_POLY(float, 1);
  } else {
    if (vec) GIBBS_POLY(bf16, 4); else GIBBS_POLY(bf16, 1);
  }
#undef GIBBS_POLY
  GIBBS_LAUNCH_STATUS("poly_norm");
}

GIBBS_EXPORT int gibbs_gemm_heads(const void* X, long ldx, long head_x, const void* W, long head_w, long ldw, void* Y, long ldy,
                                  long head_y, int dtype, int n, int O, int I, int heads, hipStream_t stream) {
  return gibbs_gemm_heads_gated(X, ldx, head_x, W, head_w, ldw, Y, ldy, head_y, nullptr, 0, 0, dtype, n, O, I, heads, stream);
}

// The per-head products with every result multiplied by sigmoid(G[n][h][o]) (G null: plain), G's rows ldg and its heads head_g apart.
GIBBS_EXPORT int gibbs_gemm_heads_gated(const void* X, long ldx, long head_x, const void* W, long head_w, long ldw, void* Y, long ldy,
                                        long head_y, const void* G, long ldg, long head_g, int dtype, int n, int O, int I, int heads,
                                        hipStream_t stream) {
  GIBBS_REQUIRE(n >= 0 && O > 0 && I > 0 && heads > 0 && heads <= 65535, "gemm_heads: bad sizes n=%d O=%d I=%d heads=%d", n, O, I, heads);
  GIBBS_REQUIRE(ldx >= I && ldw >= I && ldy >= O, "gemm_heads: row strides shorter than rows");
  if (n == 0) return 0;
  dim3 grid(ceil_div(O, 64), ceil_div(n, 64), heads);
  GIBBS_REQUIRE(grid.y <= 65535, "gemm_heads: too many rows (%d)", n);
  if (dtype == GIBBS_F32) {
    gemm_heads_plain_kernel<float><<<grid, 256, 0, stream>>>((const float*)X, ldx, head_x, (const float*)W, head_w, ldw, (float*)Y, ldy, head_y, n, O, I, (const float*)G, ldg, head_g);
  } else if (dtype == GIBBS_BF16) {
    const bool aligned = I % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && head_x % 8 == 0 && head_w % 8 == 0 && ((uintptr_t)X % 16) == 0 &&
                         ((uintptr_t)W % 16) == 0;
    // (8-byte stores and gate loads: rows, heads and the pointers themselves at multiples of 4 values)
    const bool vec = ldy % 4 == 0 && head_y % 4 == 0 && ((uintptr_t)Y % 8) == 0 &&
                     (!G || (ldg % 4 == 0 && head_g % 4 == 0 && ((uintptr_t)G % 8) == 0));
    if (aligned && vec)
      gemm_heads_mfma_kernel<true><<<grid, 256, 0, stream>>>((const bf16*)X, ldx, head_x, (const bf16*)W, head_w, ldw, (bf16*)Y, ldy, head_y, n, O, I, (const bf16*)G, ldg, head_g);
    else if (aligned)
      gemm_heads_mfma_kernel<false><<<grid, 256, 0, stream>>>((const bf16*)X, ldx, head_x, (const bf16*)W, head_w, ldw, (bf16*)Y, ldy, head_y, n, O, I, (const bf16*)G, ldg, head_g);
    else
      gemm_heads_plain_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)X, ldx, head_x, (const bf16*)W, head_w, ldw, (bf16*)Y, ldy, head_y, n, O, I, (const bf16*)G, ldg, head_g);
  } else {
    return gibbs_fail("gemm_heads: unknown dtype %d", dtype);
  }
  GIBBS_LAUNCH_STATUS("gemm_heads");
}
