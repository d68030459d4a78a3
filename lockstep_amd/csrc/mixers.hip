// Kernels of the mixers, norms and activations beyond the softmax-attention decoder: Dynamic Tanh
// norm (with the deferred residual addition), the clamped gated unit, the soft cap of the logits,
// the post pass of an attention projection with biases, partial rotation, value mixing and cache
// write for keys and values of different sizes, the linear recurrence with per-row decay and write
// gates (HGRN2, retention), and the per-head RMS norm with an optional weight and gate.
//
// Everything here is computed in float whatever the compute dtype T is: T is the type of what a
// matrix product reads next (and of the cache).  Per-row reductions have an order fixed by the
// row's sizes alone; the recurrence walks a request's tokens in order, so nothing depends on how
// the request was cut into steps or on what else is in the batch.

#include "common.h"
#include "mixers_api.h"

namespace ls {

struct SeqMeta {  // one per sequence of the step (all int32), as the step's upload lays it out
  int q_off;      // first packed row
  int q_len;      // rows in this step
  int q_start;    // absolute position of the first row
  int kv_len;     // q_start + q_len
  int table_row;  // row of the block table, and the request's state slot
  int reserved[3];
};

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x * sigmoidf_(x); }

// ---------------------------------------------------------------------------
// Dynamic Tanh norm of rows of the float residual stream, elementwise:
//   h[row] += P[0][row] + P[1][row] + ...   (when P is given; slices ascending, from +0)
//   out[r] = tanh(alpha * h[row]) * w + b
// `row` = rows[r] when a row list is given.  alpha is one float on the device.
// out == nullptr: the addition only.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void dyt_kernel(float* __restrict__ h, const float* __restrict__ P, int slices,
                                                  long p_stride, const float* __restrict__ weight,
                                                  const float* __restrict__ bias, const float* __restrict__ alpha,
                                                  T* __restrict__ out, const int* __restrict__ rows, int width,
                                                  long ldh, long ld_out) {
  const int r_out = blockIdx.x;
  const long row = rows ? rows[r_out] : r_out;
  float* src = h + row * ldh;
  const float a = out ? alpha[0] : 0.f;
  for (int e = threadIdx.x; e < width; e += 256) {
    float v = src[e];
    if (P) {
      float sum = 0.f;
      for (int s = 0; s < slices; ++s) sum = sum + P[s * p_stride + row * width + e];
      v = v + sum;
      src[e] = v;
    }
    if (out) out[(long)r_out * ld_out + e] = from_f32<T>(tanhf(a * v) * weight[e] + bias[e]);
  }
}

// ---------------------------------------------------------------------------
// Clamped gated unit on float rows x [rows][2 * width] (gates, then ups):
//   g = min(gate, limit); u = clamp(up, -limit, limit); out = g * sigmoid(alpha * g) * (u + 1)
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void glu_clamped_kernel(const float* __restrict__ x, long ldx, T* __restrict__ out,
                                                          long ldo, int rows, int width, float limit, float alpha) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)rows * width) return;
  const long r = idx / width;
  const int c = (int)(idx % width);
  const float g = fminf(x[r * ldx + c], limit);
  const float u = fminf(fmaxf(x[r * ldx + width + c], -limit), limit);
  out[r * ldo + c] = from_f32<T>((g * sigmoidf_(alpha * g)) * (u + 1.0f));
}

// Soft cap in place: x = cap * tanh(x / cap).
__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, long ld, int rows, int width, float cap) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)rows * width) return;
  float* at = x + (idx / width) * ld + idx % width;
  *at = cap * tanhf(*at / cap);
}

// ---------------------------------------------------------------------------
// Rotation of element i of a head (rot leading dimensions, pair (i, i + rot/2)) at a position.
// `own` and `other` are the element and its partner; cos/sin tables [positions][rot/2].
// ---------------------------------------------------------------------------
__device__ __forceinline__ float rotate_element(float own, float other, int i, int rot, const float* cos_row,
                                                const float* sin_row) {
  const int half = rot >> 1;
  if (i < half) return own * cos_row[i] - other * sin_row[i];
  return own * cos_row[i - half] + other * sin_row[i - half];
}

// ---------------------------------------------------------------------------
// Post pass of an attention projection raw [T][ld] float = q (H heads of D) | k (G of D) | v (G of DV):
//   biases added; q and k rotated on their first `rot` dimensions at the token's position;
//   q -> q_out [T][H*D] (T);  k -> key pages [page][G][slot][D];
//   v -> value pages [page][G][DV][slot], after value mixing:
//     mode 1: v is also kept in v_first [T][G*DV] (float) for the layers that follow;
//     mode 2: v = (1 - lambda) v + lambda v_first[t], lambda one float on the device.
// One thread per element.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void talk_qkv_kernel(
    const float* __restrict__ raw, long ld, int n_tokens, int H, int G, int D, int DV, const float* __restrict__ bias,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const SeqMeta* __restrict__ seqs, const int* __restrict__ table, int table_stride,
    T* __restrict__ q_out, long ldq, T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int vmix_mode,
    const float* __restrict__ vmix, float* __restrict__ v_first, long ldv) {
  const int width = H * D + G * D + G * DV;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)n_tokens * width) return;
  const int t = (int)(idx / width);
  const int e = (int)(idx % width);
  const float* row = raw + (long)t * ld;
  const int pos = tok_pos[t];
  float own = row[e] + (bias ? bias[e] : 0.f);
  const int qk = (H + G) * D;
  if (e < qk) {
    const int i = e % D;
    if (i < rot) {
      const int half = rot >> 1;
      const int pe = i < half ? e + half : e - half;
      const float other = row[pe] + (bias ? bias[pe] : 0.f);
      own = rotate_element(own, other, i, rot, cos_table + (long)pos * half, sin_table + (long)pos * half);
    }
    if (e < H * D) {
      q_out[(long)t * ldq + e] = from_f32<T>(own);
      return;
    }
  }
  const int table_row = seqs[tok_seq[t]].table_row;
  const int page = table[(long)table_row * table_stride + pos / page_size];
  const int slot = pos % page_size;
  if (e < qk) {
    const int g = (e - H * D) / D, i = e % D;
    if (page >= 0) k_pages[(((long)page * G + g) * page_size + slot) * D + i] = from_f32<T>(own);
    return;
  }
  const int c = e - qk;  // column of the token's values, g * DV + i
  if (vmix_mode == 1) v_first[(long)t * ldv + c] = own;
  if (vmix_mode == 2) {
    const float lam = vmix[0];
    own = (1.0f - lam) * own + lam * v_first[(long)t * ldv + c];
  }
  const int g = c / DV, i = c % DV;
  if (page >= 0) v_pages[(((long)page * G + g) * DV + i) * page_size + slot] = from_f32<T>(own);
}

// ---------------------------------------------------------------------------
// Linear recurrence with a decay and a write gate for every row of the state, one head:
//   S_t = diag(a_t) S_(t-1) + b_t v_t^T,   o_t = S_t^T q_t,     S [D][DV] float, kept per request.
// mode 0 (HGRN2): q = silu(q_raw), f = lower + (1 - lower) sigmoid(f_raw + f_bias), a = f, b = 1 - f.
// mode 1 (retention): q = rotate(q_raw), b = rotate(k_raw) D^(-1/2), a = decay[head] for every row.
// raw [T][ld] float holds q_raw at q_at, f_raw / k_raw at ab_at, v at v_at (H heads each).
//
// A workgroup takes (request, head, block of 64 columns of the state): wave g keeps the rows
// [16 g, 16 g + 16) of its column in registers, one column a lane, and walks the request's tokens
// in order, sixteen at a time: their q, a, b and v are prepared in LDS by all threads, every wave
// adds its rows' part of o_t, and the parts are added in wave order.  The order of all sums is a
// function of D alone.
// ---------------------------------------------------------------------------
constexpr int kRecRows = 16;    // rows of the state a lane keeps
constexpr int kRecTokens = 16;  // tokens prepared at a time

__global__ __launch_bounds__(1024) void linrec_kernel(
    int mode, const float* __restrict__ raw, long ld, int q_at, int ab_at, int v_at, int H, int D, int DV,
    const float* __restrict__ p0, const float* __restrict__ p1, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, const SeqMeta* __restrict__ seqs, float* __restrict__ state,
    float* __restrict__ out, long ldo) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x / H, head = blockIdx.x % H, cb = blockIdx.y;
  const SeqMeta m = seqs[seq];
  if (m.q_len <= 0) return;
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int dp = waves * kRecRows;  // D rounded up to the rows the waves hold
  float* q_s = lds;                                // [tokens][dp]
  float* a_s = q_s + kRecTokens * dp;
  float* b_s = a_s + kRecTokens * dp;
  float* v_s = b_s + kRecTokens * dp;              // [tokens][64]
  float* o_s = v_s + kRecTokens * 64;              // [waves][tokens][64]
  const int c = cb * 64 + lane;
  const bool col_ok = c < DV;
  float* mine = state + (((long)m.table_row * H + head) * D) * DV;
  float S[kRecRows];
#pragma unroll
  for (int r = 0; r < kRecRows; ++r) {
    const int row = g * kRecRows + r;
    S[r] = (row < D && col_ok) ? mine[(long)row * DV + c] : 0.f;
  }
  const float inv_sqrt_d = 1.0f / sqrtf((float)D);
  const int half = rot >> 1;
  for (int t0 = 0; t0 < m.q_len; t0 += kRecTokens) {
    const int n = min(kRecTokens, m.q_len - t0);
    for (int idx = threadIdx.x; idx < n * dp; idx += blockDim.x) {
      const int tt = idx / dp, row = idx % dp;
      float q = 0.f, a = 0.f, b = 0.f;
      if (row < D) {
        const float* src = raw + (long)(m.q_off + t0 + tt) * ld;
        const int e = head * D + row;
        if (mode == 0) {
          const float lower = p0[e];
          const float f = lower + (1.0f - lower) * sigmoidf_(src[ab_at + e] + (p1 ? p1[e] : 0.f));
          q = siluf_(src[q_at + e]);
          a = f;
          b = 1.0f - f;
        } else {
          q = src[q_at + e];
          b = src[ab_at + e];
          if (row < rot) {
            const int pe = row < half ? e + half : e - half;
            const long pos = m.q_start + t0 + tt;
            q = rotate_element(q, src[q_at + pe], row, rot, cos_table + pos * half, sin_table + pos * half);
            b = rotate_element(b, src[ab_at + pe], row, rot, cos_table + pos * half, sin_table + pos * half);
          }
          b = b * inv_sqrt_d;
          a = p0[head];
        }
      }
      q_s[idx] = q;
      a_s[idx] = a;
      b_s[idx] = b;
    }
    for (int idx = threadIdx.x; idx < n * 64; idx += blockDim.x) {
      const int tt = idx >> 6, col = cb * 64 + (idx & 63);
      v_s[idx] = col < DV ? raw[(long)(m.q_off + t0 + tt) * ld + v_at + head * DV + col] : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < n; ++tt) {
      const float v = v_s[tt * 64 + lane];
      const float* qa = q_s + tt * dp + g * kRecRows;
      const float* aa = a_s + tt * dp + g * kRecRows;
      const float* ba = b_s + tt * dp + g * kRecRows;
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < kRecRows; ++r) {
        S[r] = aa[r] * S[r] + ba[r] * v;
        o = o + S[r] * qa[r];
      }
      o_s[(g * kRecTokens + tt) * 64 + lane] = o;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < n * 64; idx += blockDim.x) {
      const int tt = idx >> 6, l = idx & 63, col = cb * 64 + l;
      float o = 0.f;
      for (int w = 0; w < waves; ++w) o = o + o_s[(w * kRecTokens + tt) * 64 + l];
      if (col < DV) out[(long)(m.q_off + t0 + tt) * ldo + head * DV + col] = o;
    }
    // (the next round's preparation writes q_s .. v_s only, which no thread reads any more; its
    // barrier stands between these reads of o_s and the next writes to it)
  }
#pragma unroll
  for (int r = 0; r < kRecRows; ++r) {
    const int row = g * kRecRows + r;
    if (row < D && col_ok) mine[(long)row * DV + c] = S[r];
  }
}

// ---------------------------------------------------------------------------
// Per (token, head): x [DV] float divided by its root mean square (eps inside the root), times
// weight[c] if given, times silu(gate[t][head * DV + c]) if given; stored as T.  One wave a
// head: lane i adds the squares of the elements i, i + 64, ... ascending, then a butterfly.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ x, long ldx, int n_tokens,
                                                             int H, int DV, const float* __restrict__ weight,
                                                             const float* __restrict__ gate, long ldg, float eps,
                                                             T* __restrict__ out, long ldo) {
  const long unit = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= (long)n_tokens * H) return;
  const int t = (int)(unit / H), head = (int)(unit % H), lane = threadIdx.x & 63;
  const float* src = x + (long)t * ldx + head * DV;
  float part = 0.f;
  for (int c = lane; c < DV; c += 64) part = part + src[c] * src[c];
  const float total = wave_sum(part);
  const float scale = 1.0f / sqrtf(total / (float)DV + eps);
  for (int c = lane; c < DV; c += 64) {
    float v = src[c] * scale;
    if (weight) v = v * weight[c];
    if (gate) v = v * siluf_(gate[(long)t * ldg + head * DV + c]);
    out[(long)t * ldo + head * DV + c] = from_f32<T>(v);
  }
}

}  // namespace ls

LS_DEFINE_ERROR_API

#define LS_MIXERS_LISTED(X) \
  X(ls_dyt) X(ls_glu_clamped) X(ls_softcap) X(ls_talk_qkv) X(ls_linrec) X(ls_head_norm_gate)
LS_DEFINE_LISTED_CALLS(LS_MIXERS_LISTED)

using namespace ls;

extern "C" int ls_dyt(int dtype, float* h, const float* P, int slices, int p_rows, const float* weight,
                      const float* bias, const float* alpha, void* out, const int* rows, int n_rows, int width,
                      long ldh, long ld_out, void* stream) {
  LS_REQUIRE(n_rows > 0 && width > 0 && ldh >= width && h, "dyt: bad sizes");
  LS_REQUIRE(!out || (weight && bias && alpha && ld_out >= width), "dyt: an output needs weight, bias and alpha");
  LS_REQUIRE(!P || (slices > 0 && p_rows > 0), "dyt: bad slice sums");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long p_stride = (long)p_rows * width;
  if (dtype == kF32)
    hipLaunchKernelGGL(dyt_kernel<float>, dim3(n_rows), dim3(256), 0, s, h, P, slices, p_stride, weight, bias, alpha,
                       (float*)out, rows, width, ldh, ld_out);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(dyt_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, s, h, P, slices, p_stride, weight, bias, alpha,
                       (bf16_t*)out, rows, width, ldh, ld_out);
  else
    return fail("dyt: unknown dtype %d", dtype);
  return check_launch("dyt");
}

extern "C" int ls_glu_clamped(int out_dtype, const float* x, long ldx, void* out, long ldo, int rows, int width,
                              float limit, float alpha, void* stream) {
  LS_REQUIRE(rows > 0 && width > 0 && ldo >= width && ldx >= 2 * width && x && out, "glu_clamped: bad sizes");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)(((long)rows * width + 255) / 256));
  if (out_dtype == kF32)
    hipLaunchKernelGGL(glu_clamped_kernel<float>, grid, dim3(256), 0, s, x, ldx, (float*)out, ldo, rows, width, limit,
                       alpha);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL(glu_clamped_kernel<bf16_t>, grid, dim3(256), 0, s, x, ldx, (bf16_t*)out, ldo, rows, width,
                       limit, alpha);
  else
    return fail("glu_clamped: unknown dtype %d", out_dtype);
  return check_launch("glu_clamped");
}

extern "C" int ls_softcap(float* x, long ld, int rows, int width, float cap, void* stream) {
  LS_REQUIRE(rows > 0 && width > 0 && ld >= width && x && cap > 0.f, "softcap: bad sizes");
  dim3 grid((unsigned)(((long)rows * width + 255) / 256));
  hipLaunchKernelGGL(softcap_kernel, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream), x, ld, rows, width,
                     cap);
  return check_launch("softcap");
}

extern "C" int ls_talk_qkv(int dtype, const float* raw, long ld, int n_tokens, int H, int G, int D, int DV,
                           const float* bias, const float* cos_table, const float* sin_table, int rot,
                           int table_positions, int max_pos, const int* tok_seq, const int* tok_pos, const void* seqs,
                           const int* table, int table_stride, void* q_out, long ldq, void* k_pages, void* v_pages,
                           int page_size, int vmix_mode, const float* vmix, float* v_first, long ldv, void* stream) {
  LS_REQUIRE(n_tokens > 0 && H > 0 && G > 0 && D > 0 && DV > 0 && H % G == 0, "talk_qkv: bad head sizes");
  const long width = (long)H * D + (long)G * D + (long)G * DV;
  LS_REQUIRE(ld >= width && ldq >= (long)H * D && raw && q_out && k_pages && v_pages && table && seqs && tok_seq &&
                 tok_pos && page_size > 0 && table_stride > 0,
             "talk_qkv: bad operands");
  LS_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D, "talk_qkv: %d rotated dimensions of %d", rot, D);
  LS_REQUIRE(rot == 0 || (cos_table && sin_table && max_pos < table_positions),
             "talk_qkv: position %d is beyond the rotation tables (%d)", max_pos, table_positions);
  LS_REQUIRE(max_pos / page_size < table_stride, "talk_qkv: position %d is beyond the block table", max_pos);
  LS_REQUIRE(vmix_mode >= 0 && vmix_mode <= 2 && (vmix_mode == 0 || (v_first && ldv >= (long)G * DV)) &&
                 (vmix_mode != 2 || vmix),
             "talk_qkv: bad value mixing");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)((n_tokens * width + 255) / 256));
#define LS_TALK_QKV(T_)                                                                                              \
  hipLaunchKernelGGL(talk_qkv_kernel<T_>, grid, dim3(256), 0, s, raw, ld, n_tokens, H, G, D, DV, bias, cos_table,    \
                     sin_table, rot, tok_seq, tok_pos, (const SeqMeta*)seqs, table, table_stride, (T_*)q_out, ldq,   \
                     (T_*)k_pages, (T_*)v_pages, page_size, vmix_mode, vmix, v_first, ldv)
  if (dtype == kF32)
    LS_TALK_QKV(float);
  else if (dtype == kBF16)
    LS_TALK_QKV(bf16_t);
  else
    return fail("talk_qkv: unknown dtype %d", dtype);
#undef LS_TALK_QKV
  return check_launch("talk_qkv");
}

extern "C" int ls_linrec_max_dim() { return 64 * kRecRows / 4; }

extern "C" int ls_linrec(int mode, const float* raw, long ld, int q_at, int ab_at, int v_at, int H, int D, int DV,
                         const float* p0, const float* p1, const float* cos_table, const float* sin_table, int rot,
                         int table_positions, int max_pos, const void* seqs, int n_seqs, float* state, float* out,
                         long ldo, void* stream) {
  LS_REQUIRE(mode == 0 || mode == 1, "linrec: unknown mode %d", mode);
  LS_REQUIRE(n_seqs > 0 && H > 0 && D > 0 && DV > 0 && D <= ls_linrec_max_dim(),
             "linrec: bad sizes (heads %d, rows %d of at most %d, columns %d)", H, D, ls_linrec_max_dim(), DV);
  LS_REQUIRE(raw && seqs && state && out && p0 && ldo >= (long)H * DV, "linrec: bad operands");
  LS_REQUIRE(q_at >= 0 && ab_at >= 0 && v_at >= 0 && ld >= q_at + (long)H * D && ld >= ab_at + (long)H * D &&
                 ld >= v_at + (long)H * DV,
             "linrec: the projections do not fit the rows");
  if (mode == 1) {
    LS_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D, "linrec: %d rotated dimensions of %d", rot, D);
    LS_REQUIRE(rot == 0 || (cos_table && sin_table && max_pos < table_positions),
               "linrec: position %d is beyond the rotation tables (%d)", max_pos, table_positions);
  }
  const int waves = (D + kRecRows - 1) / kRecRows;
  const int dp = waves * kRecRows;
  const size_t lds = sizeof(float) * (size_t)(3 * kRecTokens * dp + kRecTokens * 64 + waves * kRecTokens * 64);
  if (lds > 48 * 1024) {  // (more than the default bound of dynamic LDS: say so once a size)
    static size_t allowed = 0;
    if (lds > allowed) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(linrec_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return fail("linrec: %s", hipGetErrorString(e));
      allowed = lds;
    }
  }
  dim3 grid((unsigned)(n_seqs * H), (unsigned)((DV + 63) / 64));
  hipLaunchKernelGGL(linrec_kernel, grid, dim3(64 * waves), lds, reinterpret_cast<hipStream_t>(stream), mode, raw, ld,
                     q_at, ab_at, v_at, H, D, DV, p0, p1, cos_table, sin_table, mode == 1 ? rot : 0,
                     (const SeqMeta*)seqs, state, out, ldo);
  return check_launch("linrec");
}

extern "C" int ls_head_norm_gate(int out_dtype, const float* x, long ldx, int n_tokens, int H, int DV,
                                 const float* weight, const float* gate, long ldg, float eps, void* out, long ldo,
                                 void* stream) {
  LS_REQUIRE(n_tokens > 0 && H > 0 && DV > 0 && x && out && ldx >= (long)H * DV && ldo >= (long)H * DV &&
                 (!gate || ldg >= (long)H * DV),
             "head_norm_gate: bad sizes");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)(((long)n_tokens * H + 3) / 4));
  if (out_dtype == kF32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, dim3(256), 0, s, x, ldx, n_tokens, H, DV, weight, gate, ldg,
                       eps, (float*)out, ldo);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, dim3(256), 0, s, x, ldx, n_tokens, H, DV, weight, gate,
                       ldg, eps, (bf16_t*)out, ldo);
  else
    return fail("head_norm_gate: unknown dtype %d", out_dtype);
  return check_launch("head_norm_gate");
}
