// The operations of a Llama-style decoder layer that sit between the quantised linears, for single-token
// decode: residual add + RMSNorm, rotary embedding + KV-cache append + attention of one query token over the
// cache, SwiGLU gating, greedy pick.  Plain HBM/L2-latency-bound kernels; they exist so that a decode step is
// a short chain of launches that a HIP graph can replay, not to be clever.
#include <cstdlib>

#include "common.hpp"

namespace glowq {

namespace {

__device__ __forceinline__ float block_sum(float v, float* red, int nwaves) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  __syncthreads();  // red may still be read from a previous call
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += red[i];
  return t;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

__device__ __forceinline__ float block_max(float v, float* red, int nwaves) {
  v = wave_max(v);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = red[0];
  for (int i = 1; i < nwaves; ++i) t = fmaxf(t, red[i]);
  return t;
}

}  // namespace

// x[m] = fp16(x[m] + delta[m]) (when delta != nullptr), h[m] = fp16(x[m] * rsqrt(mean(x[m]^2) + eps) * w), one
// workgroup per token row, statistics in fp32.
__global__ __launch_bounds__(1024) void add_rmsnorm_kernel(half_t* __restrict__ x, const half_t* __restrict__ delta,
                                                            const half_t* __restrict__ w, half_t* __restrict__ h,
                                                            int H, float eps) {
  __shared__ float red[16];
  half_t* xr = x + (size_t)blockIdx.x * H;
  const half_t* dr = delta ? delta + (size_t)blockIdx.x * H : nullptr;
  half_t* hr = h + (size_t)blockIdx.x * H;
  const int nw = blockDim.x >> 6;
  float ss = 0.f;
  for (int i = threadIdx.x * 8; i < H; i += blockDim.x * 8) {  // H % 8 == 0
    h8 v = *reinterpret_cast<const h8*>(xr + i);
    if (dr) {
      const h8 d = *reinterpret_cast<const h8*>(dr + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = (half_t)((float)v[j] + (float)d[j]);
      *reinterpret_cast<h8*>(xr + i) = v;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) ss = __builtin_fmaf((float)v[j], (float)v[j], ss);
  }
  const float inv = rsqrtf(block_sum(ss, red, nw) / (float)H + eps);
  for (int i = threadIdx.x * 8; i < H; i += blockDim.x * 8) {
    const h8 v = *reinterpret_cast<const h8*>(xr + i);  // own writes of the first pass
    const h8 ww = *reinterpret_cast<const h8*>(w + i);
    h8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (half_t)((float)(half_t)((float)v[j] * inv) * (float)ww[j]);
    *reinterpret_cast<h8*>(hr + i) = o;
  }
}

// Single-token forms that also produce the shared right-factor projection of their output, so the group launch that
// follows needs no projection launch of its own.  One workgroup per row j of R: every workgroup recomputes the (cheap)
// elementwise result, dots it with R[j] and writes r[j]; the elementwise outputs are written in 8-element chunks dealt
// round robin over the workgroups.  x_out must not alias x_in (other workgroups still read it).
template <int kMax>  // chunks of 8 per thread: H <= 8 * blockDim.x * kMax
__global__ __launch_bounds__(512) void add_rmsnorm_proj_kernel(const half_t* __restrict__ x_in, const half_t* __restrict__ delta,
                                                               const half_t* __restrict__ w, half_t* __restrict__ x_out,
                                                               half_t* __restrict__ h, const half_t* __restrict__ R,
                                                               half_t* __restrict__ r, int H, int rank, float eps) {
  __shared__ float red[16];
  const int j = blockIdx.x;
  const int nw = blockDim.x >> 6;
  const int chunks = H >> 3;
  h8 xv[kMax], wv[kMax], rv[kMax];
  // every load goes out before the first reduction: one memory round trip for the whole kernel
#pragma unroll
  for (int c = 0; c < kMax; ++c) {
    const int i = min((int)(threadIdx.x + c * blockDim.x), chunks - 1);
    xv[c] = reinterpret_cast<const h8*>(x_in)[i];
    wv[c] = reinterpret_cast<const h8*>(w)[i];
    rv[c] = reinterpret_cast<const h8*>(R + (size_t)j * H)[i];
  }
  if (delta) {
    h8 dv[kMax];
#pragma unroll
    for (int c = 0; c < kMax; ++c) dv[c] = reinterpret_cast<const h8*>(delta)[min((int)(threadIdx.x + c * blockDim.x), chunks - 1)];
#pragma unroll
    for (int c = 0; c < kMax; ++c)
#pragma unroll
      for (int e = 0; e < 8; ++e) xv[c][e] = (half_t)((float)xv[c][e] + (float)dv[c][e]);
  }
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < kMax; ++c) {
    const bool live = threadIdx.x + c * blockDim.x < chunks;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = __builtin_fmaf(live ? (float)xv[c][e] : 0.f, (float)xv[c][e], ss);
  }
  const float inv = rsqrtf(block_sum(ss, red, nw) / (float)H + eps);
  float dot = 0.f;
#pragma unroll
  for (int c = 0; c < kMax; ++c) {
    const int i = threadIdx.x + c * blockDim.x;
    if (i < chunks) {
      // fp16(x * inv) in fp32, then the weight as a packed fp16 product (the fp32 product of two halves is exact, so one
      // rounding either way) and the dot with R two elements at a time in fp32
      h8 o;
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const h2 n2 = {(half_t)((float)xv[c][e] * inv), (half_t)((float)xv[c][e + 1] * inv)};
        const h2 w2 = {wv[c][e], wv[c][e + 1]};
        const h2 o2 = n2 * w2;
        o[e] = o2[0];
        o[e + 1] = o2[1];
        dot = __builtin_amdgcn_fdot2(o2, h2{rv[c][e], rv[c][e + 1]}, dot, false);
      }
      if (i % rank == j) {
        reinterpret_cast<h8*>(x_out)[i] = xv[c];
        reinterpret_cast<h8*>(h)[i] = o;
      }
    }
  }
  dot = block_sum(dot, red, nw);
  if (threadIdx.x == 0) r[j] = (half_t)dot;
}

// 1024 threads, at most kMax chunks of 8 per thread, all loads first.
template <int kMax>  // chunks of 8 per thread: n <= 8 * 1024 * kMax
__global__ __launch_bounds__(1024) void silu_mul_proj_kernel(const half_t* __restrict__ gate, const half_t* __restrict__ up,
                                                             half_t* __restrict__ out, const half_t* __restrict__ R,
                                                             half_t* __restrict__ r, int n, int rank) {
  __shared__ float red[16];
  const int j = blockIdx.x;
  const int nw = blockDim.x >> 6;
  const int chunks = n >> 3;
  h8 gv[kMax], uv[kMax], rv[kMax];
#pragma unroll
  for (int c = 0; c < kMax; ++c) {
    const int i = min((int)(threadIdx.x + c * blockDim.x), chunks - 1);
    gv[c] = reinterpret_cast<const h8*>(gate)[i];
    uv[c] = reinterpret_cast<const h8*>(up)[i];
    rv[c] = reinterpret_cast<const h8*>(R + (size_t)j * n)[i];
  }
  float dot = 0.f;
#pragma unroll
  for (int c = 0; c < kMax; ++c) {
    const int i = threadIdx.x + c * blockDim.x;
    if (i < chunks) {
      h8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float gf = (float)gv[c][e];
        o[e] = (half_t)((float)(half_t)silu_f32(gf) * (float)uv[c][e]);
        dot = __builtin_fmaf((float)o[e], (float)rv[c][e], dot);
      }
      if (i % rank == j) reinterpret_cast<h8*>(out)[i] = o;
    }
  }
  dot = block_sum(dot, red, nw);
  if (threadIdx.x == 0) r[j] = (half_t)dot;
}

// out = silu(gate) * up, elementwise, fp32 math.
__global__ __launch_bounds__(256) void silu_mul_kernel(const half_t* __restrict__ gate, const half_t* __restrict__ up,
                                                        half_t* __restrict__ out, long n8) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += (long)gridDim.x * blockDim.x) {
    const h8 g = reinterpret_cast<const h8*>(gate)[i];
    const h8 u = reinterpret_cast<const h8*>(up)[i];
    h8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float gf = (float)g[j];
      o[j] = (half_t)((float)(half_t)silu_f32(gf) * (float)u[j]);
    }
    reinterpret_cast<h8*>(out)[i] = o;
  }
}

// Sum over the kLanes (8 or 16) consecutive lanes that share a cache row; every lane of the group gets the total.
template <int kLanes>
__device__ __forceinline__ float row_group_sum(float v) {
  int t;
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, t);
  t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true);  // row_half_mirror
  v += __builtin_bit_cast(float, t);
  if constexpr (kLanes == 16) {
    t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true);  // row_mirror
    v += __builtin_bit_cast(float, t);
  }
  return v;
}

// One query token against the cache, one workgroup (8 waves by default, up to 16) per query head and split; kD = head dimension (64 or 128).
//   q [heads, d], k_new / v_new [kv_heads, d]: this token's projections (k, q not yet rotated)
//   cos / sin [max_len, d] fp32 tables (second half repeats the first), *pos the token's position
//   cache_k / cache_v [kv_heads, max_len, d] fp16: positions < pos are read; position pos is WRITTEN by the first
//   head of each KV group and taken from LDS by all, so no workgroup reads what another one writes.
//   out [heads, d] fp16.
// d/8 consecutive lanes share a cache row (16 bytes each: a wave load covers 4 or 8 whole rows, several loads in
// flight), scores go to LDS (max_len floats), softmax over [0, pos], then P.V with the same lane mapping.
template <int kD>
__global__ __launch_bounds__(1024) void rope_attend_kernel(const half_t* __restrict__ q, const half_t* __restrict__ k_new,
                                                            const half_t* __restrict__ v_new, const float* __restrict__ cos_t,
                                                            const float* __restrict__ sin_t, const long* __restrict__ pos_p,
                                                            half_t* __restrict__ cache_k, half_t* __restrict__ cache_v,
                                                            half_t* __restrict__ out, float* __restrict__ part, int heads,
                                                            int kv_heads, int max_len, float scale) {
  constexpr int d = kD;
  constexpr int kLanes = d / 8;           // lanes per cache row
  constexpr int kRowsPerWave = 64 / kLanes;
  constexpr int kUnroll = 4;
  constexpr int half_d = d >> 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  float* qs = reinterpret_cast<float*>(smem_raw);            // [d] rotated query
  float* kn = qs + d;                                        // [d] rotated key of this token
  float* vn = kn + d;                                        // [d] value of this token
  float* wave_m = vn + d;                                    // [16] running maximum of each wave
  float* wave_l = wave_m + 16;                               // [16] sum of exponentials of each wave
  float* acc_part = wave_l + 16;                             // [waves][d]
  const int head = blockIdx.x;
  const int rep = heads / kv_heads;
  const int kvh = head / rep;
  // context split: the cached positions are dealt to the gridDim.y workgroups of a head row by row, workgroup s taking
  // s, s + splits, ...; the last one also takes the token itself.  Which rows a lane reads first therefore does not
  // depend on the position, and those loads go out before anything else is known.  With a split the unnormalised
  // partial {max, sum, -, -, acc[d]} goes to `part`, else the result to `out`.
  const int splits = gridDim.y, split = blockIdx.y;
  const bool own = split == splits - 1;
  const int nw = blockDim.x >> 6;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int sub = lane % kLanes, rg = lane / kLanes;
  const int row0 = wave * kRowsPerWave + rg;      // first of this lane group's rows (counted within the workgroup)
  const int row_step = nw * kRowsPerWave;
  auto position = [&](int t) { return split + splits * t; };

  // One pass over the rows with a running maximum (no score buffer): every lane group keeps {m, l, acc[8 of its
  // dimensions]} for its own rows.  The key and the value row of a position are loaded together, one batch of kUnroll
  // rows ahead of the batch being worked on.
  const half_t* kbase = cache_k + (size_t)kvh * max_len * d + 8 * sub;
  const half_t* vbase = cache_v + (size_t)kvh * max_len * d + 8 * sub;
  struct Batch {
    h8 k[kUnroll], v[kUnroll];
  };
  auto fetch = [&](int t, Batch& bt) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const size_t off = (size_t)min(position(t + u * row_step), max_len - 1) * d;  // rows past the position go unused
      bt.k[u] = *reinterpret_cast<const h8*>(kbase + off);
      bt.v[u] = *reinterpret_cast<const h8*>(vbase + off);
    }
  };
  Batch b0, b1;
  fetch(row0, b0);
  float q0 = 0.f, q1 = 0.f, k0 = 0.f, k1 = 0.f;
  half_t v0 = (half_t)0.f, v1 = (half_t)0.f;
  if (threadIdx.x < half_d) {
    const int i = threadIdx.x;
    q0 = (float)q[(size_t)head * d + i], q1 = (float)q[(size_t)head * d + i + half_d];
    k0 = (float)k_new[(size_t)kvh * d + i], k1 = (float)k_new[(size_t)kvh * d + i + half_d];
    v0 = v_new[(size_t)kvh * d + i], v1 = v_new[(size_t)kvh * d + i + half_d];
  }
  const int pos = (int)*pos_p;
  // A position outside the cache (a caller stepping past max_len - 1): the tables and the caches are not indexed out of
  // bounds and no cache row is written; the output (or this workgroup's partial) becomes NaN, so that everything
  // computed from this step says so instead of carrying the last step's values on.  Uniform over the grid.
  if (pos < 0 || pos >= max_len) {
    const float bad = __builtin_nanf("");
    if (part) {
      float* mine = part + ((size_t)head * splits + split) * (d + 4);
      for (int i = threadIdx.x; i < d + 4; i += blockDim.x) mine[i] = bad;
    } else {
      for (int i = threadIdx.x; i < d; i += blockDim.x) out[(size_t)head * d + i] = (half_t)bad;
    }
    return;
  }

  // rotary embedding of q and k_new: out[i] = x[i] cos - x[i + d/2] sin, out[i + d/2] = x[i + d/2] cos + x[i] sin
  if (threadIdx.x < half_d) {
    const int i = threadIdx.x;
    // the tables are rounded to fp16 first, as a half-precision model's rotary embedding does
    const float c = (float)(half_t)cos_t[(size_t)pos * d + i], sn = (float)(half_t)sin_t[(size_t)pos * d + i];
    // Two fp32 products and one fp32 sum, each rounded on its own, then one rounding to fp16: what the elementwise
    // tensor expression x * cos + rotate_half(x) * sin evaluates.  A fused multiply-add skips the rounding of one
    // product, which now and then lands on the other side of an fp16 rounding boundary (one cached key element in some
    // thousand rows differed by an fp16 ulp from the tensor expression before contraction was switched off here).
    float qa, qb, ka, kb;
    {
#pragma clang fp contract(off)
      const float q0c = q0 * c, q1s = q1 * sn, q1c = q1 * c, q0s = q0 * sn;
      const float k0c = k0 * c, k1s = k1 * sn, k1c = k1 * c, k0s = k0 * sn;
      qa = q0c - q1s;
      qb = q1c + q0s;
      ka = k0c - k1s;
      kb = k1c + k0s;
    }
    qs[i] = (float)(half_t)qa;
    qs[i + half_d] = (float)(half_t)qb;
    const half_t r0 = (half_t)ka, r1 = (half_t)kb;
    kn[i] = (float)r0;
    kn[i + half_d] = (float)r1;
    vn[i] = (float)v0;
    vn[i + half_d] = (float)v1;
    if (head == kvh * rep && split == 0) {
      half_t* ck = cache_k + ((size_t)kvh * max_len + pos) * d;
      half_t* cv = cache_v + ((size_t)kvh * max_len + pos) * d;
      ck[i] = r0; ck[i + half_d] = r1;
      cv[i] = v0; cv[i + half_d] = v1;
    }
  }
  __syncthreads();

  float qv[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) qv[j] = qs[8 * sub + j];

  float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) acc[j] = 0.f;
  auto fold = [&](int t, const Batch& bt) {
    float sv[kUnroll];
    float bm = m;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float dot = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) dot = __builtin_fmaf(qv[j], (float)bt.k[u][j], dot);
      dot = row_group_sum<kLanes>(dot);
      sv[u] = (position(t + u * row_step) < pos) ? dot * scale : -INFINITY;
      bm = fmaxf(bm, sv[u]);
    }
    // the first row of a batch is always a real one, so bm is finite here
    const float keep = __expf(m - bm);
    l *= keep;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] *= keep;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const float e = __expf(sv[u] - bm);
      l += e;
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] = __builtin_fmaf(e, (float)bt.v[u][j], acc[j]);
    }
    m = bm;
  };
  {
    const int step = kUnroll * row_step;
    int t = row0;
    while (position(t) < pos) {
      const int t1 = t + step;
      if (position(t1) < pos) fetch(t1, b1);
      fold(t, b0);
      if (position(t1) >= pos) break;
      const int t2 = t1 + step;
      if (position(t2) < pos) fetch(t2, b0);
      fold(t1, b1);
      t = t2;
    }
  }
  if (wave == 0 && rg == 0 && own) {  // this token against itself
    float dot = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) dot = __builtin_fmaf(qv[j], kn[8 * sub + j], dot);
    const float sv = row_group_sum<kLanes>(dot) * scale;
    const float bm = fmaxf(m, sv);
    const float keep = __expf(m - bm), e = __expf(sv - bm);
    l = l * keep + e;
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = __builtin_fmaf(e, vn[8 * sub + j], acc[j] * keep);
    m = bm;
  }
  // the lane groups of a wave meet through lane exchanges, the waves through LDS
  {
    float mw = m;
#pragma unroll
    for (int o = kLanes; o < 64; o <<= 1) mw = fmaxf(mw, __shfl_xor(mw, o));
    const float keep = (m == -INFINITY) ? 0.f : __expf(m - mw);
    l *= keep;
#pragma unroll
    for (int o = kLanes; o < 64; o <<= 1) l += __shfl_xor(l, o);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      acc[j] *= keep;
#pragma unroll
      for (int o = kLanes; o < 64; o <<= 1) acc[j] += __shfl_xor(acc[j], o);
    }
    if (rg == 0) {
#pragma unroll
      for (int j = 0; j < 8; ++j) acc_part[wave * d + 8 * sub + j] = acc[j];
      if (sub == 0) {
        wave_m[wave] = mw;
        wave_l[wave] = l;
      }
    }
  }
  __syncthreads();
  // the waves' partials meet: the first nw lanes of wave 0 turn the waves' maxima into weights (and the sum of the
  // weighted sums), then one thread per dimension adds the weighted accumulators
  if (wave == 0) {
    const float mw = lane < nw ? wave_m[lane] : -INFINITY;
    float mx = mw;
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    const float wgt = (mw == -INFINITY) ? 0.f : __expf(mw - mx);
    float sum = lane < nw ? wave_l[lane] * wgt : 0.f;
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) sum += __shfl_xor(sum, o);
    if (lane < nw) wave_m[lane] = wgt;  // from here on: the wave's weight
    if (lane == 0) {
      wave_l[0] = sum;
      wave_l[1] = mx;
    }
  }
  __syncthreads();
  float* mine = part ? part + ((size_t)head * splits + split) * (d + 4) : nullptr;
  const float sum = wave_l[0];
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float t = 0.f;
    for (int w = 0; w < nw; ++w) t = __builtin_fmaf(acc_part[w * d + i], wave_m[w], t);
    if (part) mine[4 + i] = t;
    else out[(size_t)head * d + i] = (half_t)(t / sum);
  }
  if (part && threadIdx.x == 0) {
    mine[0] = wave_l[1];  // -inf for a split without rows: its weight in the combination is exp(-inf) = 0
    mine[1] = sum;
  }
}

// Combines the split partials of rope_attend_kernel into out [heads * d] fp16 and, with R, also computes the shared
// projection r[j] = out . R[j] of the group that consumes it: one workgroup per row of R recomputes the combination
// (the partials are a few tens of KB) and writes 8-element chunks of `out` dealt round robin, as the other fused
// glue kernels do.  Without R a few workgroups just write their chunks.
template <int kCombineSplits>  // splits whose partials are all fetched before any is used (more walk them one by one)
__global__ __launch_bounds__(1024) void attend_combine_proj_kernel(const float* __restrict__ part, half_t* __restrict__ out,
                                                                   const half_t* __restrict__ R, half_t* __restrict__ r,
                                                                   int heads, int d, int splits) {
  __shared__ float red[16];
  const int j = blockIdx.x, nwg = gridDim.x;
  const int n = heads * d, chunks = n >> 3;
  const int nw = blockDim.x >> 6;
  const int stride = d + 4;
  float dot = 0.f;
  for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
    const int head = (c << 3) / d, i0 = (c << 3) - head * d;
    const float* ph = part + (size_t)head * splits * stride;
    h8 rr;
    if (R) rr = reinterpret_cast<const h8*>(R + (size_t)j * n)[c];
    float mx = -INFINITY, den = 0.f, acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    if (splits <= kCombineSplits) {
      float pm[kCombineSplits], pl[kCombineSplits];
      f4 lo[kCombineSplits], hi[kCombineSplits];
#pragma unroll
      for (int s = 0; s < kCombineSplits; ++s) {
        const float* ps = ph + min(s, splits - 1) * stride;
        pm[s] = s < splits ? ps[0] : -INFINITY;
        pl[s] = ps[1];
        lo[s] = *reinterpret_cast<const f4*>(ps + 4 + i0);
        hi[s] = *reinterpret_cast<const f4*>(ps + 8 + i0);
      }
#pragma unroll
      for (int s = 0; s < kCombineSplits; ++s) mx = fmaxf(mx, pm[s]);
#pragma unroll
      for (int s = 0; s < kCombineSplits; ++s) {
        const float w = (pm[s] == -INFINITY) ? 0.f : __expf(pm[s] - mx);
        den = __builtin_fmaf(w, pl[s], den);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc[e] = __builtin_fmaf(w, lo[s][e], acc[e]);
          acc[4 + e] = __builtin_fmaf(w, hi[s][e], acc[4 + e]);
        }
      }
    } else {
      for (int s = 0; s < splits; ++s) mx = fmaxf(mx, ph[s * stride]);
      for (int s = 0; s < splits; ++s) {
        const float pm = ph[s * stride];
        const float w = (pm == -INFINITY) ? 0.f : __expf(pm - mx);
        den = __builtin_fmaf(w, ph[s * stride + 1], den);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(w, ph[s * stride + 4 + i0 + e], acc[e]);
      }
    }
    const float inv = __builtin_amdgcn_rcpf(den);
    h8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (half_t)(acc[e] * inv);
    if (R) {
#pragma unroll
      for (int e = 0; e < 8; ++e) dot = __builtin_fmaf((float)o[e], (float)rr[e], dot);
    }
    if (c % nwg == j) reinterpret_cast<h8*>(out)[c] = o;
  }
  if (R) {
    dot = block_sum(dot, red, nw);
    if (threadIdx.x == 0) r[j] = (half_t)dot;
  }
}

// Index of the first maximum of an fp16 vector, one workgroup; then token <- index, position += 1.
__global__ __launch_bounds__(1024) void argmax_advance_kernel(const half_t* __restrict__ logits, int n, long* __restrict__ next_tok,
                                                               long* __restrict__ tok, long* __restrict__ pos) {
  __shared__ float bv[16];
  __shared__ int bi[16];
  float best = -INFINITY;
  int idx = 0x7fffffff;
  const int n8 = (reinterpret_cast<uintptr_t>(logits) & 15) == 0 ? n / 8 : 0;  // 16-byte pieces, then the tail
  // batches of eight pieces per thread, all requested before the first is looked at: a round trip per batch, not per piece
  constexpr int kBatch = 8;
  for (int i0 = threadIdx.x; i0 < n8; i0 += kBatch * blockDim.x) {
    h8 v[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) v[b] = reinterpret_cast<const h8*>(logits)[min(i0 + b * (int)blockDim.x, n8 - 1)];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int i = i0 + b * (int)blockDim.x;
      if (i < n8) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if ((float)v[b][j] > best) {  // ascending index per thread: the first maximum wins
            best = (float)v[b][j];
            idx = 8 * i + j;
          }
      }
    }
  }
  for (int i = 8 * n8 + threadIdx.x; i < n; i += blockDim.x) {
    const float v = (float)logits[i];
    if (v > best || (v == best && i < idx)) {
      best = v;
      idx = i;
    }
  }
#pragma unroll
  for (int o = 32; o; o >>= 1) {
    const float ov = __shfl_xor(best, o);
    const int oi = __shfl_xor(idx, o);
    if (ov > best || (ov == best && oi < idx)) {
      best = ov;
      idx = oi;
    }
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  if (lane == 0) {
    bv[wave] = best;
    bi[wave] = idx;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < idx)) {
        best = bv[w];
        idx = bi[w];
      }
    *next_tok = idx;
    if (tok) *tok = idx;
    if (pos) *pos += 1;
  }
}

// ---- launchers ------------------------------------------------------------------------------
hipError_t launch_add_rmsnorm(half_t* x, const half_t* delta, const half_t* w, half_t* h, int M, int H, float eps,
                              hipStream_t stream) {
  int threads = ((H / 8 + 63) / 64) * 64;
  if (threads > 1024) threads = 1024;
  if (threads < 64) threads = 64;
  hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(M), dim3(threads), 0, stream, x, delta, w, h, H, eps);
  return hipGetLastError();
}

hipError_t launch_silu_mul(const half_t* gate, const half_t* up, half_t* out, long n, int num_cus, hipStream_t stream) {
  const long n8 = n / 8;
  long blocks = (n8 + 255) / 256;
  if (blocks > (long)num_cus * 8) blocks = (long)num_cus * 8;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, gate, up, out, n8);
  return hipGetLastError();
}

hipError_t launch_add_rmsnorm_proj(const half_t* x_in, const half_t* delta, const half_t* w, half_t* x_out, half_t* h,
                                   const half_t* R, half_t* r, int H, int rank, float eps, hipStream_t stream) {
  // 512 threads and as few chunk slots per thread as H needs: every workgroup redoes the whole elementwise part, so
  // slots that only repeat the last chunk are instructions on its critical path
  const int slots = ((H >> 3) + 511) / 512;
  if (slots <= 1)
    hipLaunchKernelGGL(add_rmsnorm_proj_kernel<1>, dim3(rank), dim3(512), 0, stream, x_in, delta, w, x_out, h, R, r, H, rank, eps);
  else if (slots == 2)
    hipLaunchKernelGGL(add_rmsnorm_proj_kernel<2>, dim3(rank), dim3(512), 0, stream, x_in, delta, w, x_out, h, R, r, H, rank, eps);
  else
    hipLaunchKernelGGL(add_rmsnorm_proj_kernel<4>, dim3(rank), dim3(512), 0, stream, x_in, delta, w, x_out, h, R, r, H, rank, eps);
  return hipGetLastError();
}

hipError_t launch_silu_mul_proj(const half_t* gate, const half_t* up, half_t* out, const half_t* R, half_t* r, int n, int rank,
                                hipStream_t stream) {
  const int slots = ((n >> 3) + 1023) / 1024;
  if (slots <= 1)
    hipLaunchKernelGGL(silu_mul_proj_kernel<1>, dim3(rank), dim3(1024), 0, stream, gate, up, out, R, r, n, rank);
  else if (slots == 2)
    hipLaunchKernelGGL(silu_mul_proj_kernel<2>, dim3(rank), dim3(1024), 0, stream, gate, up, out, R, r, n, rank);
  else
    hipLaunchKernelGGL(silu_mul_proj_kernel<4>, dim3(rank), dim3(1024), 0, stream, gate, up, out, R, r, n, rank);
  return hipGetLastError();
}

size_t rope_attend_lds(int d, int max_len) {
  (void)max_len;  // no per-position buffer: the context length is bounded by the cache alone
  return (size_t)(3 * d + 32 + 16 * d) * sizeof(float);
}

template <int kD>
static hipError_t launch_rope_attend_t(const half_t* q, const half_t* k_new, const half_t* v_new, const float* cos_t,
                                       const float* sin_t, const long* pos, half_t* cache_k, half_t* cache_v, half_t* out,
                                       float* part, int splits, int heads, int kv_heads, int max_len, float scale,
                                       hipStream_t stream) {
  const size_t lds = rope_attend_lds(kD, max_len);
  static LdsLimit lds_limit;
  if (hipError_t e = ensure_dynamic_lds(reinterpret_cast<const void*>(rope_attend_kernel<kD>), lds, lds_limit); e != hipSuccess) return e;
  static const int env_threads = getenv("GLOWQ_ATTEND_THREADS") ? atoi(getenv("GLOWQ_ATTEND_THREADS")) : 0;
  // eight waves per workgroup: the decode step at 575 cached positions reads 1.847 ms per token with 16 waves, 1.835 with 4,
  // 1.827 with 6, 1.822 with 8, 1.823 with 10, 1.832 with 12 (a 1024-thread workgroup has the compute unit to itself)
  const int threads = (env_threads >= 64 && env_threads <= 1024 && env_threads % 64 == 0) ? env_threads : 512;
  hipLaunchKernelGGL(rope_attend_kernel<kD>, dim3(heads, splits), dim3(threads), lds, stream, q, k_new, v_new,
                     cos_t, sin_t, pos, cache_k, cache_v, out, part, heads, kv_heads, max_len, scale);
  return hipGetLastError();
}

hipError_t launch_rope_attend(const half_t* q, const half_t* k_new, const half_t* v_new, const float* cos_t,
                              const float* sin_t, const long* pos, half_t* cache_k, half_t* cache_v, half_t* out, float* part,
                              int splits, int heads, int kv_heads, int d, int max_len, float scale, hipStream_t stream) {
  if (d == 128)
    return launch_rope_attend_t<128>(q, k_new, v_new, cos_t, sin_t, pos, cache_k, cache_v, out, part, splits, heads, kv_heads,
                                     max_len, scale, stream);
  if (d == 64)
    return launch_rope_attend_t<64>(q, k_new, v_new, cos_t, sin_t, pos, cache_k, cache_v, out, part, splits, heads, kv_heads,
                                    max_len, scale, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_attend_combine_proj(const float* part, half_t* out, const half_t* R, half_t* r, int heads, int d, int splits,
                                      int rank, hipStream_t stream) {
  const int wgs = R ? rank : 32;
  const int chunks = heads * d / 8;
  int threads = (chunks + 63) / 64 * 64;  // one 8-element chunk per thread where the workgroup size allows
  threads = threads < 64 ? 64 : (threads > 1024 ? 1024 : threads);
  if (splits <= 2)
    hipLaunchKernelGGL(attend_combine_proj_kernel<2>, dim3(wgs), dim3(threads), 0, stream, part, out, R, r, heads, d, splits);
  else if (splits <= 4)
    hipLaunchKernelGGL(attend_combine_proj_kernel<4>, dim3(wgs), dim3(threads), 0, stream, part, out, R, r, heads, d, splits);
  else
    hipLaunchKernelGGL(attend_combine_proj_kernel<8>, dim3(wgs), dim3(threads), 0, stream, part, out, R, r, heads, d, splits);
  return hipGetLastError();
}

hipError_t launch_argmax_advance(const half_t* logits, int n, long* next_tok, long* tok, long* pos, hipStream_t stream) {
  hipLaunchKernelGGL(argmax_advance_kernel, dim3(1), dim3(1024), 0, stream, logits, n, next_tok, tok, pos);
  return hipGetLastError();
}

}  // namespace glowq

using namespace glowq;

extern "C" {

int glowq_add_rmsnorm(void* x, const void* delta, const void* weight, void* h, int M, int H, float eps, void* stream) {
  if (!x || !weight || !h) return fail(GLOWQ_EINVAL, "add_rmsnorm: x, weight and h must be device pointers");
  if (M <= 0 || H <= 0 || (H & 7)) return fail(GLOWQ_EINVAL, "add_rmsnorm: M > 0 and H a positive multiple of 8 (got M=%d, H=%d)", M, H);
  hipError_t e = launch_add_rmsnorm(static_cast<half_t*>(x), static_cast<const half_t*>(delta), static_cast<const half_t*>(weight),
                                    static_cast<half_t*>(h), M, H, eps, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? GLOWQ_OK : fail(GLOWQ_ELAUNCH, "add_rmsnorm launch failed: %s", hipGetErrorString(e));
}

int glowq_silu_mul(const void* gate, const void* up, void* out, long n, void* stream) {
  if (!gate || !up || !out) return fail(GLOWQ_EINVAL, "silu_mul: gate, up and out must be device pointers");
  if (n <= 0 || (n & 7)) return fail(GLOWQ_EINVAL, "silu_mul: n must be a positive multiple of 8 (got %ld)", n);
  hipError_t e = launch_silu_mul(static_cast<const half_t*>(gate), static_cast<const half_t*>(up), static_cast<half_t*>(out), n,
                                 num_cus(), static_cast<hipStream_t>(stream));
  return e == hipSuccess ? GLOWQ_OK : fail(GLOWQ_ELAUNCH, "silu_mul launch failed: %s", hipGetErrorString(e));
}

int glowq_add_rmsnorm_proj(const void* x_in, const void* delta, const void* weight, void* x_out, void* h, const void* R,
                           void* r, int H, int rank, float eps, void* stream) {
  if (!x_in || !weight || !x_out || !h || !R || !r) return fail(GLOWQ_EINVAL, "add_rmsnorm_proj: pointers must be device pointers");
  if (x_in == x_out) return fail(GLOWQ_EINVAL, "add_rmsnorm_proj: x_out must not alias x_in");
  if (H <= 0 || (H & 7) || H > 8192 || rank <= 0)
    return fail(GLOWQ_EINVAL, "add_rmsnorm_proj: H a multiple of 8 up to 8192 and rank > 0 (got H=%d, rank=%d)", H, rank);
  hipError_t e = launch_add_rmsnorm_proj(static_cast<const half_t*>(x_in), static_cast<const half_t*>(delta),
                                         static_cast<const half_t*>(weight), static_cast<half_t*>(x_out), static_cast<half_t*>(h),
                                         static_cast<const half_t*>(R), static_cast<half_t*>(r), H, rank, eps,
                                         static_cast<hipStream_t>(stream));
  return e == hipSuccess ? GLOWQ_OK : fail(GLOWQ_ELAUNCH, "add_rmsnorm_proj launch failed: %s", hipGetErrorString(e));
}

int glowq_silu_mul_proj(const void* gate, const void* up, void* out, const void* R, void* r, int n, int rank, void* stream) {
  if (!gate || !up || !out || !R || !r) return fail(GLOWQ_EINVAL, "silu_mul_proj: pointers must be device pointers");
  if (n <= 0 || (n & 7) || n > 32768 || rank <= 0)
    return fail(GLOWQ_EINVAL, "silu_mul_proj: n a multiple of 8 up to 32768, rank > 0 (got %d, %d)", n, rank);
  hipError_t e = launch_silu_mul_proj(static_cast<const half_t*>(gate), static_cast<const half_t*>(up), static_cast<half_t*>(out),
                                      static_cast<const half_t*>(R), static_cast<half_t*>(r), n, rank, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? GLOWQ_OK : fail(GLOWQ_ELAUNCH, "silu_mul_proj launch failed: %s", hipGetErrorString(e));
}

int glowq_rope_attend(const void* q, const void* k_new, const void* v_new, const float* cos_table, const float* sin_table,
                      const int64_t* pos, void* cache_k, void* cache_v, void* out, int heads, int kv_heads, int head_dim,
                      int max_len, float scale, void* stream) {
  if (!q || !k_new || !v_new || !cos_table || !sin_table || !pos || !cache_k || !cache_v || !out)
    return fail(GLOWQ_EINVAL, "rope_attend: all pointers must be device pointers");
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || max_len <= 0)
    return fail(GLOWQ_EINVAL, "rope_attend: heads must be a positive multiple of kv_heads (got %d, %d)", heads, kv_heads);
  if (head_dim != 64 && head_dim != 128) return fail(GLOWQ_EUNSUPPORTED, "rope_attend: head_dim must be 64 or 128 (got %d)", head_dim);
  hipError_t e = launch_rope_attend(static_cast<const half_t*>(q), static_cast<const half_t*>(k_new), static_cast<const half_t*>(v_new),
                                    cos_table, sin_table, reinterpret_cast<const long*>(pos), static_cast<half_t*>(cache_k),
                                    static_cast<half_t*>(cache_v), static_cast<half_t*>(out), nullptr, 1, heads, kv_heads, head_dim,
                                    max_len, scale, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? GLOWQ_OK : fail(GLOWQ_ELAUNCH, "rope_attend launch failed: %s", hipGetErrorString(e));
}

int glowq_rope_attend_split(const void* q, const void* k_new, const void* v_new, const float* cos_table, const float* sin_table,
                            const int64_t* pos, void* cache_k, void* cache_v, float* partials, int splits, int heads,
                            int kv_heads, int head_dim, int max_len, float scale, void* stream) {
  if (!q || !k_new || !v_new || !cos_table || !sin_table || !pos || !cache_k || !cache_v || !partials)
    return fail(GLOWQ_EINVAL, "rope_attend_split: all pointers must be device pointers");
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || max_len <= 0 || splits < 1 || splits > 64)
    return fail(GLOWQ_EINVAL, "rope_attend_split: heads a positive multiple of kv_heads, 1..64 splits (got %d, %d, %d)", heads,
                kv_heads, splits);
  if (head_dim != 64 && head_dim != 128)
    return fail(GLOWQ_EUNSUPPORTED, "rope_attend_split: head_dim must be 64 or 128 (got %d)", head_dim);
  hipError_t e = launch_rope_attend(static_cast<const half_t*>(q), static_cast<const half_t*>(k_new), static_cast<const half_t*>(v_new),
                                    cos_table, sin_table, reinterpret_cast<const long*>(pos), static_cast<half_t*>(cache_k),
                                    static_cast<half_t*>(cache_v), nullptr, partials, splits, heads, kv_heads, head_dim, max_len,
                                    scale, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? GLOWQ_OK : fail(GLOWQ_ELAUNCH, "rope_attend_split launch failed: %s", hipGetErrorString(e));
}

int glowq_attend_combine_proj(const float* partials, void* out, const void* R, void* r, int heads, int head_dim, int splits,
                              int rank, void* stream) {
  if (!partials || !out) return fail(GLOWQ_EINVAL, "attend_combine_proj: partials and out must be device pointers");
  if ((R == nullptr) != (r == nullptr)) return fail(GLOWQ_EINVAL, "attend_combine_proj: R and r go together");
  if (heads <= 0 || head_dim <= 0 || (head_dim & 7) || splits < 1 || (R && rank <= 0))
    return fail(GLOWQ_EINVAL, "attend_combine_proj: bad sizes (heads %d, head_dim %d, splits %d, rank %d)", heads, head_dim, splits, rank);
  hipError_t e = launch_attend_combine_proj(partials, static_cast<half_t*>(out), static_cast<const half_t*>(R), static_cast<half_t*>(r),
                                            heads, head_dim, splits, rank, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? GLOWQ_OK : fail(GLOWQ_ELAUNCH, "attend_combine_proj launch failed: %s", hipGetErrorString(e));
}

int glowq_argmax_advance(const void* logits, int n, int64_t* next_token, int64_t* token, int64_t* pos, void* stream) {
  if (!logits || !next_token || n <= 0) return fail(GLOWQ_EINVAL, "argmax_advance: logits and next_token must be device pointers, n > 0");
  hipError_t e = launch_argmax_advance(static_cast<const half_t*>(logits), n, reinterpret_cast<long*>(next_token),
                                       reinterpret_cast<long*>(token), reinterpret_cast<long*>(pos), static_cast<hipStream_t>(stream));
  return e == hipSuccess ? GLOWQ_OK : fail(GLOWQ_ELAUNCH, "argmax_advance launch failed: %s", hipGetErrorString(e));
}

}  // extern "C"
