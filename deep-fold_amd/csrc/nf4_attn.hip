// Decode attention for gfx950: split-KV flash-decode over the valid prefix of a
// static bf16 KV cache with fused rotate-half RoPE and cache write, the merge of
// the split partials, and the standalone RoPE + cache write.
// Replaces chr_nf4_attn / chr_nf4_rope_kv (gpu/nf4/nf4_gemv.cu:497-727, 926-994).
//
// One 64-lane wavefront serves one (query head, split).  A cache row of hd
// values is read by LPT = hd/8 lanes with one 16-byte load each, so a wavefront
// walks 64/LPT time steps per iteration (four at hd = 128); each lane group
// keeps its own online-softmax state and the groups are folded once at the end.
// Split s owns the time steps t with t % n_split == s.
//
// Numerics (gpu/nf4/nf4_gemv.cu:599-727): the rotated query and the rotated
// current key stay fp32; older keys and all values come from the bf16 cache;
// running max starts at -1e30; exp is the fast hardware exponential.

#include <cstdlib>

#include "nf4_common.h"

namespace chr {
namespace {

constexpr float kNegBig = -1.0e30f;

__device__ __forceinline__ void widen8(const uint4 v, float *f) {
  f[0] = bf16_lo(v.x);
  f[1] = bf16_hi(v.x);
  f[2] = bf16_lo(v.y);
  f[3] = bf16_hi(v.y);
  f[4] = bf16_lo(v.z);
  f[5] = bf16_hi(v.z);
  f[6] = bf16_lo(v.w);
  f[7] = bf16_hi(v.w);
}

__device__ __forceinline__ uint4 narrow8(const float *f) {
  uint4 v;
  v.x = f32_to_bf16(f[0]) | (static_cast<uint32_t>(f32_to_bf16(f[1])) << 16);
  v.y = f32_to_bf16(f[2]) | (static_cast<uint32_t>(f32_to_bf16(f[3])) << 16);
  v.z = f32_to_bf16(f[4]) | (static_cast<uint32_t>(f32_to_bf16(f[5])) << 16);
  v.w = f32_to_bf16(f[6]) | (static_cast<uint32_t>(f32_to_bf16(f[7])) << 16);
  return v;
}

// Rotate-half on the eight dims [d0, d0+8) of a head vector `t` (bf16 in
// memory), fp32 result.  half = hd/2; d0 is a multiple of 8 and so never
// straddles the half boundary.  out[d] = t[d]*cos[d] - t[d+half]*sin[d] for
// d < half, t[d]*cos[d] + t[d-half]*sin[d] otherwise.
__device__ __forceinline__ void rope8(const uint16_t *t, const uint16_t *cos, const uint16_t *sin,
                                      int d0, int half, float *out) {
  float a[8], b[8], c[8], s[8];
  const bool low = d0 < half;
  const int partner = low ? d0 + half : d0 - half;
  widen8(*reinterpret_cast<const uint4 *>(t + d0), a);
  widen8(*reinterpret_cast<const uint4 *>(t + partner), b);
  widen8(*reinterpret_cast<const uint4 *>(cos + d0), c);
  widen8(*reinterpret_cast<const uint4 *>(sin + d0), s);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float rot = low ? -b[i] : b[i];
    out[i] = a[i] * c[i] + rot * s[i];
  }
}

struct AttnArgs {
  const uint16_t *q;
  const uint16_t *k_cache;
  const uint16_t *v_cache;
  float *m_s;
  float *l_s;
  float *o_s;
  const int32_t *valid_len;
  const uint16_t *k_act;
  const uint16_t *v_act;
  const uint16_t *cos;
  const uint16_t *sin;
  const int64_t *position;
  int n_q, n_kv, hd, n_split, max_seq;
  float scale;
  uint16_t *out;  // merged heads, bf16 [n_q, hd]
  // one-workgroup forms: n_parts workgroups per head (>= 1); with state != nullptr each
  // leaves its unnormalised softmax state {m, l, 0, 0, o[hd]} at state[(head*n_parts+part)]
  // for a later merge instead of writing out
  int n_parts;
  float *state;
  // several query tokens in one launch (blockIdx.y = token): token t reads its q at
  // q + t*q_tok_stride, sees *valid_len + t cache rows, and writes dim d of a head to
  // out[t*out_tok_stride + (head*hd + d)*out_dim_stride]
  int q_tok_stride, out_tok_stride, out_dim_stride;
  // one-workgroup forms: workgroups are dealt to the eight dies of the chip in turn (workgroup
  // b runs on die b % 8, each with its own L2).  With xcd_map the (head, part) of a workgroup
  // follows from b so that the query heads of one KV head that walk the same cache rows (the
  // same part) share a die: a cache row is then fetched from memory by one L2 instead of by
  // each die that holds one of those heads.  Placement only: what a (head, part) computes and
  // where it writes does not change.
  int xcd_map;
  // n_q / n_kv, and reciprocals for the index arithmetic ahead of the first cache request
  int n_rep;
  float inv_rep, inv_parts;
  // wavefronts of a workgroup (the block size is a hidden kernel argument: read from there it
  // is a second trip to the scalar cache ahead of the first cache request)
  int wg_waves;
};

constexpr int kDies = 8;

// (head, part) of workgroup b of a one-workgroup-form launch (n_q * n_parts workgroups a
// token).  xcd_map: die X = b % 8 holds the (KV head, part) pairs c = X, X + 8, .. (c = KV
// head * n_parts + part), each with its n_rep query heads next to each other.
// x / d for the small non-negative indices of a launch, d also given as 1.f / d: three vector
// instructions where the integer division is some thirty, on the way to a kernel's first
// memory request.  Exact for x < 2^22 and d <= 256 (every such pair checked on the CPU: (x + 0.5)
// / d is at least 0.5 / d from the next integer, the float error far below that); the host
// passes inv_d = 0 outside that range and the integer division runs.
__device__ __forceinline__ int small_div(int x, int d, float inv_d) {
  return inv_d != 0.f ? static_cast<int>((static_cast<float>(x) + 0.5f) * inv_d) : x / d;
}

__device__ __forceinline__ void locate_head(const AttnArgs &a, int b, int &head, int &part, int &kv_head) {
  if (a.xcd_map) {
    const int die = b % kDies, idx = b / kDies;
    const int j = small_div(idx, a.n_rep, a.inv_rep), r = idx - j * a.n_rep;
    const int c = die + kDies * j;
    kv_head = small_div(c, a.n_parts, a.inv_parts);
    part = c - kv_head * a.n_parts;
    head = kv_head * a.n_rep + r;
  } else {
    head = small_div(b, a.n_parts, a.inv_parts);
    part = b - head * a.n_parts;
    kv_head = small_div(head, a.n_rep, a.inv_rep);
  }
}

constexpr int kMaxWgSplits = 16;  // wavefronts of a one-workgroup-per-head launch

// out[head] = sum_s a_s o_s / sum_s a_s l_s with a_s = exp(m_s - max m); an
// empty split has m = -1e30 and l = 0, so its weight underflows to zero.
// One wavefront per head.  Lane s first takes split s's (m, l) so the maximum
// and the denominator are wavefront reductions; then every lane owns dims
// l, l+64, .. and walks the splits with all loads independent (unrolled), the
// sum over splits running in split order.
__device__ __forceinline__ void merge_head(const float *m_s, const float *l_s, const float *o_s,
                                           uint16_t *out, int head, int hd, int n_split,
                                           int lane, float *state = nullptr, int dstride = 1) {
  const float *mh = m_s + static_cast<size_t>(head) * n_split;
  const float *lh = l_s + static_cast<size_t>(head) * n_split;
  const float my_m = lane < n_split ? *(mh + lane) : kNegBig;
  const float my_l = lane < n_split ? *(lh + lane) : 0.f;
  float m = my_m;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    m = fmaxf(m, __shfl_xor(m, off, kWave));
  }
  const float my_w = __expf(my_m - m);  // weight of split `lane`
  float l = my_w * my_l;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    l += __shfl_xor(l, off, kWave);
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  const float *oh = o_s + static_cast<size_t>(head) * n_split * hd;
  uint16_t *dst = out + static_cast<size_t>(head) * hd;
  if (state != nullptr && lane == 0) {
    state[0] = m;
    state[1] = l;
  }
  // Every lane runs every iteration (the shuffles below read other lanes);
  // lanes past hd only skip the memory accesses.
  for (int d0 = 0; d0 < hd; d0 += kWave) {
    const int d = d0 + lane;
    const bool on = d < hd;
    float acc = 0.f;
    int s = 0;
    for (; s + 8 <= n_split; s += 8) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[j] = on ? *(oh + static_cast<size_t>(s + j) * hd + d) : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        acc += __shfl(my_w, s + j, kWave) * v[j];
      }
    }
    for (; s < n_split; ++s) {
      const float v = on ? *(oh + static_cast<size_t>(s) * hd + d) : 0.f;
      acc += __shfl(my_w, s, kWave) * v;
    }
    if (on) {
      if (state != nullptr) {
        state[4 + d] = acc;  // unnormalised: the later merge divides
      } else {
        dst[static_cast<size_t>(d) * dstride] = f32_to_bf16(l > 0.f ? acc * inv : 0.f);
      }
    }
  }
}

// Fold the kWave / LPT lane groups of a wavefront: lanes with equal lane % LPT hold online-softmax
// states (m, l, acc[8]) of different time-step subsets; afterwards every lane holds the state of
// their union.  (The row-swap instructions in place of the shuffles for offsets 16 and 32 were
// measured: no faster.)
template <int LPT>
__device__ __forceinline__ void fold_lane_groups(float &m, float &l, float (&acc)[8]) {
  if constexpr (LPT < kWave) {
    float mg = m;
#pragma unroll
    for (int off = LPT; off < kWave; off <<= 1) {
      mg = fmaxf(mg, __shfl_xor(mg, off, kWave));
    }
    const float w = __expf(m - mg);
    l *= w;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      acc[i] *= w;
    }
#pragma unroll
    for (int off = LPT; off < kWave; off <<= 1) {
      l += __shfl_xor(l, off, kWave);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        acc[i] += __shfl_xor(acc[i], off, kWave);
      }
    }
    m = mg;
  }
}

// The same merge for states that sit in LDS, by the workgroup that left them there (after its
// barrier): thread d takes dim d and walks the n <= 16 states itself, in state order -- no
// cross-lane traffic, every read independent -- instead of one wavefront doing the whole head
// with a shuffle per state and dim (1.3 us of a 5.3 us launch at 8 states of 128 dims; this
// form 0.3).  m and l of the states are broadcast reads; every thread computes the same
// weights.
template <int NMAX = kMaxWgSplits>  // the most states there can be
__device__ __forceinline__ void merge_wg(const float *sm, const float *sl, const float *so,
                                         uint16_t *dst, int hd, int n, int d, float *state,
                                         int dstride) {
  float m = kNegBig;
#pragma unroll
  for (int s = 0; s < NMAX; ++s) {
    m = fmaxf(m, sm[min(s, n - 1)]);
  }
  float l = 0.f, acc = 0.f;
  for (int s0 = 0; s0 < n; s0 += 8) {
    float w[8], v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int sc = min(s0 + j, n - 1);
      w[j] = s0 + j < n ? __expf(sm[sc] - m) : 0.f;
      v[j] = so[sc * hd + d];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int sc = min(s0 + j, n - 1);
      l = fmaf(w[j], sl[sc], l);
      acc = fmaf(w[j], v[j], acc);
    }
  }
  if (state != nullptr) {
    if (d == 0) {
      state[0] = m;
      state[1] = l;
    }
    state[4 + d] = acc;  // unnormalised: the later merge divides
  } else {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    dst[static_cast<size_t>(d) * dstride] = f32_to_bf16(l > 0.f ? acc * inv : 0.f);
  }
}

// LPT lanes per time step, 8 dims per lane: hd == 8*LPT.
// INWG == false: one wavefront per (head, split), partials to global memory, merged by a
//                second launch (attn_merge).
// INWG == true : one workgroup per head, wavefront w takes split w of n_split =
//                blockDim.x/64 <= 16, partials meet in LDS and the workgroup merges them:
//                no workspace and no second launch.  WMAX = the most wavefronts a workgroup of
//                the instantiation is launched with: up to 8 leave every lane 256 registers,
//                enough to hold the next block of cache rows while the current one is
//                computed (at 2047 rows an iteration took 1.5 us, 0.7 of arithmetic after
//                0.8 of waiting for its rows: 11.2 -> 10.2 us).
template <int LPT, bool INWG, int WMAX = kMaxWgSplits>
__global__ __launch_bounds__(INWG ? kWave * WMAX : kWave) void attn_flash(const AttnArgs a) {
  constexpr int TPW = kWave / LPT;  // time steps per wavefront iteration
  constexpr bool AHEAD = INWG && WMAX <= 8;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int wg_waves = a.wg_waves;
  const int n_rep = a.n_rep;
  int part = 0, head = static_cast<int>(blockIdx.x) / a.n_split, kv_head;
  if constexpr (INWG) {
    locate_head(a, static_cast<int>(blockIdx.x), head, part, kv_head);
  } else {
    kv_head = head / n_rep;
  }
  const int split = INWG ? part * wg_waves + wave : static_cast<int>(blockIdx.x) % a.n_split;
  const int lane = threadIdx.x & (kWave - 1);
  const int li = lane % LPT;  // which 8 dims of the head
  const int grp = lane / LPT; // which time step of the iteration
  const int hd = a.hd;
  const int d0 = li * 8;
  const int tok = INWG ? static_cast<int>(blockIdx.y) : 0;
  const int vl = min(*a.valid_len + tok, a.max_seq);

  // The first block of cache rows is requested before anything else (RoPE tables, q, the
  // current k/v): its trip to memory overlaps that prologue.  UNR time steps per lane group
  // and iteration: their loads are independent and all in flight together, so the trip count
  // (and with it the exposed memory latency) shrinks; the one-workgroup form has fewer
  // wavefronts per head and unrolls further.
  // (with a block read ahead, two: 5.8 / 9.8 us at 640 / 2047 rows with four, 5.4 / 9.5 with two,
  // 5.55 / 12.3 with one)
  constexpr int UNR = INWG && !AHEAD ? 4 : 2;
  const int stride = a.n_split * TPW;
  const size_t row_stride = static_cast<size_t>(a.n_kv) * hd;
  // plain dwords: arrays of vector structs would not stay in registers
  uint32_t kraw[UNR][4], vraw[UNR][4];
  // AHEAD: a second register set, so that the next block is in flight while one is computed
  uint32_t knext[AHEAD ? UNR : 1][4], vnext[AHEAD ? UNR : 1][4];
  // Every request is unconditional (a row index past `limit` reads row limit - 1 again, and the
  // values are dropped below, live[]): under a branch the number of requests in flight would
  // be unknown and every wait for an older block a wait for all of them.
  auto load_block = [&](auto &kraw, auto &vraw, int t0, int limit) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      // (the row at *position may be mid-write: it is replaced below)
      const int t = max(min(t0 + grp * a.n_split + u * stride, limit - 1), 0);
      const size_t off =
          static_cast<size_t>(t) * row_stride + static_cast<size_t>(kv_head) * hd + d0;
      const uint4 kv = *reinterpret_cast<const uint4 *>(a.k_cache + off);
      const uint4 vv = *reinterpret_cast<const uint4 *>(a.v_cache + off);
      kraw[u][0] = kv.x;
      kraw[u][1] = kv.y;
      kraw[u][2] = kv.z;
      kraw[u][3] = kv.w;
      vraw[u][0] = vv.x;
      vraw[u][1] = vv.y;
      vraw[u][2] = vv.z;
      vraw[u][3] = vv.w;
    }
  };
  // The first block is bounded by the cache size, a launch argument, not by the valid
  // length, a device scalar: its requests leave with the first instructions of the kernel
  // instead of after a round trip for that scalar.  Rows past the valid length are
  // allocated memory with arbitrary contents; they are dropped below (live[]) unused.
  load_block(kraw, vraw, split, a.max_seq);

  float qf[8];
  float kcur[8];
  float vcur[8];
  int pos = -1;
  bool fuse = false;
  const uint16_t *qh = a.q + static_cast<size_t>(tok) * a.q_tok_stride + static_cast<size_t>(head) * hd;
  bool rotated = false;
  if (a.cos != nullptr && a.sin != nullptr && a.position != nullptr) {
    const long long p = *a.position;
    if (p >= 0 && p < a.max_seq) {
      pos = static_cast<int>(p);
      const uint16_t *c = a.cos + static_cast<size_t>(pos) * hd;
      const uint16_t *s = a.sin + static_cast<size_t>(pos) * hd;
      rope8(qh, c, s, d0, hd / 2, qf);
      rotated = true;
      if (a.k_act != nullptr && a.v_act != nullptr) {
        fuse = true;
        const uint16_t *ka = a.k_act + static_cast<size_t>(kv_head) * hd;
        const uint16_t *va = a.v_act + static_cast<size_t>(kv_head) * hd;
        rope8(ka, c, s, d0, hd / 2, kcur);
        const uint4 vraw = *reinterpret_cast<const uint4 *>(va + d0);
        widen8(vraw, vcur);
        // Exactly one wavefront per KV head stores the new cache row.
        if (head == kv_head * n_rep && split == pos % a.n_split && grp == 0) {
          const size_t off = (static_cast<size_t>(pos) * a.n_kv + kv_head) * hd + d0;
          *reinterpret_cast<uint4 *>(const_cast<uint16_t *>(a.k_cache) + off) = narrow8(kcur);
          *reinterpret_cast<uint4 *>(const_cast<uint16_t *>(a.v_cache) + off) = vraw;
        }
      }
    }
  }
  if (!rotated) {
    widen8(*reinterpret_cast<const uint4 *>(qh + d0), qf);
  }

  float m = kNegBig;
  float l = 0.f;
  float acc[8] = {};
  // one block of rows (UNR slots of TPW time steps) into the running state
  auto take_block = [&](auto &kraw, auto &vraw, int t0) {
    bool live[UNR], cur[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int t = t0 + grp * a.n_split + u * stride;
      live[u] = t < vl;
      cur[u] = fuse && t == pos;
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      // the rows of slot u start at t0 + u * stride for the wavefront's first lane group: past
      // the valid length no lane has a live row in this slot or a later one (a scalar branch;
      // at 640 rows the second round of 512 keeps one slot of four)
      if (t0 + u * stride >= vl) {
        break;
      }
      float kf[8], vf[8];
      widen8(make_uint4(kraw[u][0], kraw[u][1], kraw[u][2], kraw[u][3]), kf);
      widen8(make_uint4(vraw[u][0], vraw[u][1], vraw[u][2], vraw[u][3]), vf);
      if (cur[u]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          kf[i] = kcur[i];
          vf[i] = vcur[i];
        }
      }
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        dot = fmaf(qf[i], kf[i], dot);
      }
      dot = group_sum<LPT>(dot) * a.scale;
      if (live[u]) {
        const float m2 = fmaxf(m, dot);
        const float alpha = __expf(m - m2);
        const float e = __expf(dot - m2);
        // (explicit fused multiply-adds: written a * b + c * d the compiler chooses per kernel
        // which product to fuse, and the chunk kernel must round exactly like this one)
        l = fmaf(l, alpha, e);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          acc[i] = fmaf(e, vf[i], acc[i] * alpha);
        }
        m = m2;
      }
    }
  };
  const int step = UNR * stride;
  if constexpr (AHEAD) {
    // (two blocks ahead, the loop written out over three named buffers, was slower: 6.8 / 11.0 us
    // at 640 / 2047 rows against 6.4 / 10.2 on the same box)
    for (int t0 = split; t0 < vl; t0 += step) {
      load_block(knext, vnext, t0 + step, vl);
      take_block(kraw, vraw, t0);
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          kraw[u][i] = knext[u][i];
          vraw[u][i] = vnext[u][i];
        }
      }
    }
  } else {
    for (int t0 = split; t0 < vl; t0 += step) {
      if (t0 != split) {
        load_block(kraw, vraw, t0, vl);
      }
      take_block(kraw, vraw, t0);
    }
  }

  fold_lane_groups<LPT>(m, l, acc);

  if constexpr (INWG) {
    __shared__ float sm[kMaxWgSplits], sl[kMaxWgSplits];
    __shared__ __align__(16) float so[kMaxWgSplits * 8 * LPT];
    if (lane == 0) {
      sm[wave] = m;
      sl[wave] = l;
    }
    if (grp == 0) {
      float *oh = so + wave * hd + d0;
      *reinterpret_cast<float4 *>(oh) = make_float4(acc[0], acc[1], acc[2], acc[3]);
      *reinterpret_cast<float4 *>(oh + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
    }
    __syncthreads();
    float *st = a.state == nullptr
                    ? nullptr
                    : a.state + (static_cast<size_t>(head) * a.n_parts + part) * (hd + 4);
    uint16_t *dst = a.out + static_cast<size_t>(tok) * a.out_tok_stride +
                    static_cast<size_t>(head) * hd * a.out_dim_stride;
    for (int d = threadIdx.x; d < hd; d += wg_waves * kWave) {
      merge_wg<WMAX>(sm, sl, so, dst, hd, wg_waves, d, st, a.out_dim_stride);
    }
  } else {
    const size_t slot = static_cast<size_t>(head) * a.n_split + split;
    if (lane == 0) {
      a.m_s[slot] = m;
      a.l_s[slot] = l;
    }
    if (grp == 0) {
      float *oh = a.o_s + slot * hd + d0;
      *reinterpret_cast<float4 *>(oh) = make_float4(acc[0], acc[1], acc[2], acc[3]);
      *reinterpret_cast<float4 *>(oh + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
    }
  }
}

// Chunk attention that shares the cache between the query heads of a KV head: one workgroup
// per (KV head, token), REP = n_q / n_kv query heads each.  A cache row is loaded once and
// dotted with all REP queries, so L2 traffic (what bounds a chunk: n_q * N workgroups re-read
// the prefix) drops by REP.  Rows, update order, lane-group fold and LDS merge are those of
// attn_flash<LPT, true> for each head, so a head's output is bit for bit the same.
constexpr int kMaxGqaWaves = 8;

template <int LPT, int REP>
__global__ __launch_bounds__(kWave * kMaxGqaWaves) void attn_chunk_gqa(const AttnArgs a) {
  constexpr int TPW = kWave / LPT;
  constexpr int UNR = 2;  // (4: the same within 0.5% on a prefill, 8: 1 to 5% slower)
  constexpr int HD = 8 * LPT;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int wg_waves = a.wg_waves;
  const int kv_head = static_cast<int>(blockIdx.x);
  const int tok = static_cast<int>(blockIdx.y);
  const int lane = threadIdx.x & (kWave - 1);
  const int li = lane % LPT;
  const int grp = lane / LPT;
  const int d0 = li * 8;
  const int vl = min(*a.valid_len + tok, a.max_seq);
  const int stride = wg_waves * TPW;
  const size_t row_stride = static_cast<size_t>(a.n_kv) * HD;

  // Two register sets: the block after the one being multiplied is already on its way.  The
  // requests are unconditional (rows past the prefix are clamped to its last row and masked
  // by `live` below), so the wait before the arithmetic counts exactly the newer block.
  struct Block {
    uint32_t k[UNR][4], v[UNR][4];
  };
  auto load_block = [&](Block &b, int t0) {
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      const int t = max(min(t0 + grp * wg_waves + u * stride, vl - 1), 0);  // vl may be 0
      const size_t off =
          static_cast<size_t>(t) * row_stride + static_cast<size_t>(kv_head) * HD + d0;
      const uint4 kv = *reinterpret_cast<const uint4 *>(a.k_cache + off);
      const uint4 vv = *reinterpret_cast<const uint4 *>(a.v_cache + off);
      b.k[u][0] = kv.x;
      b.k[u][1] = kv.y;
      b.k[u][2] = kv.z;
      b.k[u][3] = kv.w;
      b.v[u][0] = vv.x;
      b.v[u][1] = vv.y;
      b.v[u][2] = vv.z;
      b.v[u][3] = vv.w;
    }
  };
  Block cur, nxt;
  load_block(cur, wave);

  float qf[REP][8];
  const uint16_t *qh = a.q + static_cast<size_t>(tok) * a.q_tok_stride +
                       static_cast<size_t>(kv_head) * REP * HD + d0;
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    widen8(*reinterpret_cast<const uint4 *>(qh + r * HD), qf[r]);
  }
  float m[REP], l[REP], acc[REP][8];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    m[r] = kNegBig;
    l[r] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      acc[r][i] = 0.f;
    }
  }
  for (int t0 = wave; t0 < vl; t0 += UNR * stride) {
    load_block(nxt, t0 + UNR * stride);
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
      if (t0 + u * stride >= vl) {  // no live row in this slot or a later one, for any lane
        break;
      }
      const bool live = t0 + grp * wg_waves + u * stride < vl;
      float kf[8], vf[8];
      widen8(make_uint4(cur.k[u][0], cur.k[u][1], cur.k[u][2], cur.k[u][3]), kf);
      widen8(make_uint4(cur.v[u][0], cur.v[u][1], cur.v[u][2], cur.v[u][3]), vf);
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          dot = fmaf(qf[r][i], kf[i], dot);
        }
        dot = group_sum<LPT>(dot) * a.scale;
        if (live) {
          const float m2 = fmaxf(m[r], dot);
          const float alpha = __expf(m[r] - m2);
          const float e = __expf(dot - m2);
          l[r] = fmaf(l[r], alpha, e);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            acc[r][i] = fmaf(e, vf[i], acc[r][i] * alpha);
          }
          m[r] = m2;
        }
      }
    }
    cur = nxt;
  }

  __shared__ float sm[REP][kMaxGqaWaves], sl[REP][kMaxGqaWaves];
  __shared__ __align__(16) float so[REP][kMaxGqaWaves * HD];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    fold_lane_groups<LPT>(m[r], l[r], acc[r]);  // (different time steps, same dims)
    if (lane == 0) {
      sm[r][wave] = m[r];
      sl[r][wave] = l[r];
    }
    if (grp == 0) {
      float *oh = so[r] + wave * HD + d0;
      *reinterpret_cast<float4 *>(oh) = make_float4(acc[r][0], acc[r][1], acc[r][2], acc[r][3]);
      *reinterpret_cast<float4 *>(oh + 4) = make_float4(acc[r][4], acc[r][5], acc[r][6], acc[r][7]);
    }
  }
  __syncthreads();
  for (int item = threadIdx.x; item < REP * HD; item += wg_waves * kWave) {
    const int r = item / HD, d = item - r * HD;
    uint16_t *dst = a.out + static_cast<size_t>(tok) * a.out_tok_stride +
                    static_cast<size_t>(kv_head * REP + r) * HD * a.out_dim_stride;
    merge_wg<kMaxGqaWaves>(sm[r], sl[r], so[r], dst, HD, wg_waves, d, nullptr, a.out_dim_stride);
  }
}

template <int LPT>
bool launch_chunk_gqa(const AttnArgs &a, int n_rep, int n_waves, int n_tok, hipStream_t st) {
  const dim3 grid(static_cast<unsigned>(a.n_kv), static_cast<unsigned>(n_tok));
  const dim3 block(static_cast<unsigned>(kWave * n_waves));
  switch (n_rep) {
    case 2: attn_chunk_gqa<LPT, 2><<<grid, block, 0, st>>>(a); return true;
    case 4: attn_chunk_gqa<LPT, 4><<<grid, block, 0, st>>>(a); return true;
    case 5: attn_chunk_gqa<LPT, 5><<<grid, block, 0, st>>>(a); return true;
    case 6: attn_chunk_gqa<LPT, 6><<<grid, block, 0, st>>>(a); return true;
    case 8: attn_chunk_gqa<LPT, 8><<<grid, block, 0, st>>>(a); return true;
    default: return false;
  }
}

// Any hd <= 256: lane l owns dims l, l+64, l+128, l+192; one time step per
// iteration.  Slow path for head sizes that are not 8 * 2^n.
template <bool INWG>
__global__ __launch_bounds__(INWG ? kWave * kMaxWgSplits : kWave) void attn_flash_generic(
    const AttnArgs a) {
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int wg_waves = a.wg_waves;
  const int n_rep = a.n_rep;
  int part = 0, head = static_cast<int>(blockIdx.x) / a.n_split, kv_head;
  if constexpr (INWG) {
    locate_head(a, static_cast<int>(blockIdx.x), head, part, kv_head);
  } else {
    kv_head = head / n_rep;
  }
  const int split = INWG ? part * wg_waves + wave : static_cast<int>(blockIdx.x) % a.n_split;
  const int lane = threadIdx.x & (kWave - 1);
  const int hd = a.hd;
  const int half = hd / 2;
  const int tok = INWG ? static_cast<int>(blockIdx.y) : 0;
  const int vl = min(*a.valid_len + tok, a.max_seq);
  const uint16_t *qh = a.q + static_cast<size_t>(tok) * a.q_tok_stride + static_cast<size_t>(head) * hd;

  float qf[4] = {}, kcur[4] = {}, vcur[4] = {};
  int pos = -1;
  bool fuse = false;
  bool rotated = false;
  if (a.cos != nullptr && a.sin != nullptr && a.position != nullptr) {
    const long long p = *a.position;
    if (p >= 0 && p < a.max_seq) {
      pos = static_cast<int>(p);
      rotated = true;
      const uint16_t *c = a.cos + static_cast<size_t>(pos) * hd;
      const uint16_t *s = a.sin + static_cast<size_t>(pos) * hd;
      fuse = a.k_act != nullptr && a.v_act != nullptr;
      const uint16_t *ka = fuse ? a.k_act + static_cast<size_t>(kv_head) * hd : nullptr;
      const uint16_t *va = fuse ? a.v_act + static_cast<size_t>(kv_head) * hd : nullptr;
      const bool writer = fuse && head == kv_head * n_rep && split == pos % a.n_split;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = lane + 64 * i;
        if (d < hd) {
          const bool low = d < half;
          const int pd = low ? d + half : d - half;
          const float cd = bf16_to_f32(c[d]), sd = bf16_to_f32(s[d]);
          const float tq = bf16_to_f32(qh[d]), pq = bf16_to_f32(qh[pd]);
          qf[i] = tq * cd + (low ? -pq : pq) * sd;
          if (fuse) {
            const float tk = bf16_to_f32(ka[d]), pk = bf16_to_f32(ka[pd]);
            kcur[i] = tk * cd + (low ? -pk : pk) * sd;
            vcur[i] = bf16_to_f32(va[d]);
            if (writer) {
              const size_t off = (static_cast<size_t>(pos) * a.n_kv + kv_head) * hd + d;
              const_cast<uint16_t *>(a.k_cache)[off] = f32_to_bf16(kcur[i]);
              const_cast<uint16_t *>(a.v_cache)[off] = va[d];
            }
          }
        }
      }
    }
  }
  if (!rotated) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < hd) {
        qf[i] = bf16_to_f32(qh[d]);
      }
    }
  }

  float m = kNegBig, l = 0.f;
  float acc[4] = {};
  const size_t row_stride = static_cast<size_t>(a.n_kv) * hd;
  for (int t = split; t < vl; t += a.n_split) {
    const bool cur = fuse && t == pos;
    const size_t off = static_cast<size_t>(t) * row_stride + static_cast<size_t>(kv_head) * hd;
    float kf[4] = {}, vf[4] = {};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < hd) {
        kf[i] = cur ? kcur[i] : bf16_to_f32(a.k_cache[off + d]);
        vf[i] = cur ? vcur[i] : bf16_to_f32(a.v_cache[off + d]);
      }
    }
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dot = fmaf(qf[i], kf[i], dot);
    }
    dot = wave_sum(dot) * a.scale;
    const float m2 = fmaxf(m, dot);
    const float alpha = __expf(m - m2);
    const float e = __expf(dot - m2);
    l = fmaf(l, alpha, e);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc[i] = fmaf(e, vf[i], acc[i] * alpha);
    }
    m = m2;
  }
  if constexpr (INWG) {
    __shared__ float sm[kMaxWgSplits], sl[kMaxWgSplits];
    __shared__ float so[kMaxWgSplits * 256];
    if (lane == 0) {
      sm[wave] = m;
      sl[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < hd) {
        so[wave * hd + d] = acc[i];
      }
    }
    __syncthreads();
    float *st = a.state == nullptr
                    ? nullptr
                    : a.state + (static_cast<size_t>(head) * a.n_parts + part) * (hd + 4);
    uint16_t *dst = a.out + static_cast<size_t>(tok) * a.out_tok_stride +
                    static_cast<size_t>(head) * hd * a.out_dim_stride;
    for (int d = threadIdx.x; d < hd; d += wg_waves * kWave) {
      merge_wg(sm, sl, so, dst, hd, wg_waves, d, st, a.out_dim_stride);
    }
  } else {
    const size_t slot = static_cast<size_t>(head) * a.n_split + split;
    if (lane == 0) {
      a.m_s[slot] = m;
      a.l_s[slot] = l;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < hd) {
        a.o_s[slot * hd + d] = acc[i];
      }
    }
  }
}

// The split merge as its own launch (the two-launch form of chr_nf4_attn).
__global__ __launch_bounds__(kWave) void attn_merge(const float *__restrict__ m_s,
                                                    const float *__restrict__ l_s,
                                                    const float *__restrict__ o_s,
                                                    uint16_t *__restrict__ out, int hd,
                                                    int n_split) {
  merge_head(m_s, l_s, o_s, out, blockIdx.x, hd, n_split, threadIdx.x);
}

// Standalone RoPE + cache write: one wavefront per head (q heads first, then kv).
__global__ __launch_bounds__(kWave) void rope_kv(uint16_t *__restrict__ q, uint16_t *__restrict__ k,
                                                 const uint16_t *__restrict__ v,
                                                 uint16_t *__restrict__ k_cache,
                                                 uint16_t *__restrict__ v_cache,
                                                 const uint16_t *__restrict__ cos,
                                                 const uint16_t *__restrict__ sin,
                                                 const int64_t *__restrict__ position, int n_q,
                                                 int n_kv, int hd, int max_seq) {
  const long long p = *position;
  if (p < 0 || p >= max_seq) {
    return;
  }
  const int pos = static_cast<int>(p);
  const int hid = blockIdx.x;
  const bool is_q = hid < n_q;
  const int head = is_q ? hid : hid - n_q;
  uint16_t *vec = (is_q ? q : k) + static_cast<size_t>(head) * hd;
  const uint16_t *c = cos + static_cast<size_t>(pos) * hd;
  const uint16_t *s = sin + static_cast<size_t>(pos) * hd;
  const int half = hd / 2;
  // Read both halves before either is overwritten.
  float lo[2], hi[2];
  for (int i = 0; i < 2; ++i) {
    const int d = threadIdx.x + 64 * i;
    if (d < half) {
      const float t0 = bf16_to_f32(vec[d]);
      const float t1 = bf16_to_f32(vec[d + half]);
      lo[i] = t0 * bf16_to_f32(c[d]) + (-t1) * bf16_to_f32(s[d]);
      hi[i] = t1 * bf16_to_f32(c[d + half]) + t0 * bf16_to_f32(s[d + half]);
    }
  }
  const size_t off = (static_cast<size_t>(pos) * n_kv + head) * hd;
  for (int i = 0; i < 2; ++i) {
    const int d = threadIdx.x + 64 * i;
    if (d < half) {
      const uint16_t a = f32_to_bf16(lo[i]);
      const uint16_t b = f32_to_bf16(hi[i]);
      vec[d] = a;
      vec[d + half] = b;
      if (!is_q) {
        k_cache[off + d] = a;
        k_cache[off + d + half] = b;
        v_cache[off + d] = v[static_cast<size_t>(head) * hd + d];
        v_cache[off + d + half] = v[static_cast<size_t>(head) * hd + d + half];
      }
    }
  }
}

}  // namespace
}  // namespace chr

using namespace chr;

extern "C" int chr_nf4_rope_kv(void *q, void *k, const void *v, void *k_cache, void *v_cache,
                               const void *cos, const void *sin, const void *position,
                               int32_t n_q, int32_t n_kv, int32_t hd, int32_t max_seq,
                               void *stream) {
  if (q == nullptr || k == nullptr || v == nullptr || k_cache == nullptr || v_cache == nullptr ||
      cos == nullptr || sin == nullptr || position == nullptr) {
    return -1;
  }
  if (n_q < 1 || n_kv < 1 || hd < 2 || (hd & 1) != 0 || hd > 256 || max_seq < 1) {
    return -3;
  }
  rope_kv<<<dim3(static_cast<unsigned>(n_q + n_kv)), dim3(kWave), 0,
            static_cast<hipStream_t>(stream)>>>(
      static_cast<uint16_t *>(q), static_cast<uint16_t *>(k), static_cast<const uint16_t *>(v),
      static_cast<uint16_t *>(k_cache), static_cast<uint16_t *>(v_cache),
      static_cast<const uint16_t *>(cos), static_cast<const uint16_t *>(sin),
      static_cast<const int64_t *>(position), n_q, n_kv, hd, max_seq);
  return launch_rc();
}

namespace chr {
namespace {

template <bool INWG>
void launch_flash(const AttnArgs &a, bool vec_ok, hipStream_t st, int n_tok = 1) {
  // one-workgroup forms: a.n_split counts all wavefronts of a head (parts x wavefronts)
  const dim3 grid(static_cast<unsigned>(INWG ? a.n_q * a.n_parts : a.n_q * a.n_split),
                  static_cast<unsigned>(INWG ? n_tok : 1));
  const dim3 block(static_cast<unsigned>(INWG ? kWave * (a.n_split / a.n_parts) : kWave));
  const bool few = INWG && block.x <= 8 * kWave;  // the form that reads a block ahead
  if (vec_ok && a.hd == 128) {
    if (few) {
      attn_flash<16, INWG, 8><<<grid, block, 0, st>>>(a);
    } else {
      attn_flash<16, INWG><<<grid, block, 0, st>>>(a);
    }
  } else if (vec_ok && a.hd == 64) {
    if (few) {
      attn_flash<8, INWG, 8><<<grid, block, 0, st>>>(a);
    } else {
      attn_flash<8, INWG><<<grid, block, 0, st>>>(a);
    }
  } else if (vec_ok && a.hd == 256) {
    attn_flash<32, INWG><<<grid, block, 0, st>>>(a);
  } else if (vec_ok && a.hd == 32) {
    attn_flash<4, INWG><<<grid, block, 0, st>>>(a);
  } else if (vec_ok && a.hd == 16) {
    attn_flash<2, INWG><<<grid, block, 0, st>>>(a);
  } else {
    attn_flash_generic<INWG><<<grid, block, 0, st>>>(a);
  }
}

// mode 0: one wavefront per (head, split) + merge launch (ws = partials).
// mode 1: one workgroup of n_split wavefronts per head, merged in LDS, writes out.
// mode 2: n_parts workgroups of n_split wavefronts per head; each leaves its softmax state
//         in ws (n_q * n_parts * (hd + 4) floats) for the consumer to merge.
int attn_common(const void *q, const void *k, const void *v, void *out, const void *valid_len,
                float *ws, int32_t n_q, int32_t n_kv, int32_t hd, int32_t n_split, float scale,
                void *stream, const void *k_act, const void *v_act, const void *cos,
                const void *sin, const void *position, int32_t max_seq, int mode,
                int32_t n_parts, int32_t n_tok = 1, int32_t out_tok_stride = 0,
                int32_t out_dim_stride = 1) {
  if (q == nullptr || k == nullptr || v == nullptr || valid_len == nullptr ||
      (mode != 2 && out == nullptr) || (mode != 1 && ws == nullptr)) {
    return -1;
  }
  if (n_q < 1 || n_kv < 1 || hd < 1 || hd > 256 || (n_q % n_kv) != 0 || n_split < 1 ||
      n_split > (mode == 0 ? 64 : kMaxWgSplits) || max_seq < 1 ||
      (mode == 2 && (n_parts < 1 || n_parts > 64)) || n_tok < 1 || n_tok > 65535 ||
      (n_tok > 1 && mode != 1)) {
    return -3;
  }
  const bool rope = cos != nullptr && sin != nullptr && position != nullptr;
  if (rope && (hd & 1) != 0) {
    return -3;
  }
  if (mode == 2 && !aligned16(ws)) {
    return -5;
  }
  AttnArgs a{};
  a.q = static_cast<const uint16_t *>(q);
  a.k_cache = static_cast<const uint16_t *>(k);
  a.v_cache = static_cast<const uint16_t *>(v);
  a.n_parts = mode == 2 ? n_parts : 1;
  a.n_split = mode == 2 ? n_split * n_parts : n_split;  // wavefronts that share a head
  a.wg_waves = mode == 0 ? 1 : n_split;
  if (mode == 0) {
    const int nml = n_q * n_split;
    a.m_s = ws;
    a.l_s = ws + nml;
    a.o_s = ws + 2 * static_cast<size_t>(nml);
  } else if (mode == 2) {
    a.state = ws;
  }
  a.valid_len = static_cast<const int32_t *>(valid_len);
  a.k_act = static_cast<const uint16_t *>(k_act);
  a.v_act = static_cast<const uint16_t *>(v_act);
  a.cos = static_cast<const uint16_t *>(cos);
  a.sin = static_cast<const uint16_t *>(sin);
  a.position = static_cast<const int64_t *>(position);
  a.n_q = n_q;
  a.n_kv = n_kv;
  a.hd = hd;
  a.max_seq = max_seq;
  a.scale = scale;
  a.out = static_cast<uint16_t *>(out);
  a.q_tok_stride = n_q * hd;
  a.out_tok_stride = out_tok_stride;
  a.out_dim_stride = out_dim_stride;
  // heads that share cache rows on one die, where the (KV head, part) pairs deal out evenly
  // over the dies (CHR_ATTN_XCD_MAP=0: workgroups in head order, for comparison)
  static const bool xcd_map_on = [] {
    const char *e = std::getenv("CHR_ATTN_XCD_MAP");
    return e == nullptr || e[0] != '0';
  }();
  a.xcd_map = (xcd_map_on && mode != 0 && (n_kv * a.n_parts) % kDies == 0) ? 1 : 0;
  a.n_rep = n_q / n_kv;
  const bool small = static_cast<long long>(n_q) * a.n_parts < (1 << 22) && a.n_rep <= 256 && a.n_parts <= 256;
  a.inv_rep = small ? 1.f / static_cast<float>(a.n_rep) : 0.f;
  a.inv_parts = small ? 1.f / static_cast<float>(a.n_parts) : 0.f;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // The vector path needs 16-byte aligned rows and 16-byte aligned fp32 partials.
  const bool vec_ok = aligned16(q) && aligned16(k) && aligned16(v) &&
                      (k_act == nullptr || aligned16(k_act)) &&
                      (v_act == nullptr || aligned16(v_act)) &&
                      (cos == nullptr || aligned16(cos)) && (sin == nullptr || aligned16(sin)) &&
                      (mode != 0 || aligned16(a.o_s));
  // a chunk (several tokens) of a grouped-query model: share each cache row between the
  // query heads of its KV head when a kernel for the head size and group size exists
  bool shared = false;
  if (mode == 1 && n_tok > 1 && !rope && vec_ok && n_split <= kMaxGqaWaves) {
    const int n_rep = n_q / n_kv;
    if (hd == 128) {
      shared = launch_chunk_gqa<16>(a, n_rep, n_split, n_tok, st);
    } else if (hd == 64) {
      shared = launch_chunk_gqa<8>(a, n_rep, n_split, n_tok, st);
    }
  }
  if (shared) {
    // launched above
  } else if (mode != 0) {
    launch_flash<true>(a, vec_ok, st, n_tok);
  } else {
    launch_flash<false>(a, vec_ok, st);
    attn_merge<<<dim3(static_cast<unsigned>(n_q)), dim3(kWave), 0, st>>>(a.m_s, a.l_s, a.o_s, a.out,
                                                                         hd, n_split);
  }
  return launch_rc();
}

}  // namespace
}  // namespace chr

extern "C" int chr_nf4_attn(const void *q, const void *k, const void *v, void *out,
                            const void *valid_len, float *ws, int32_t n_q, int32_t n_kv,
                            int32_t hd, int32_t n_split, float scale, void *stream,
                            const void *k_act, const void *v_act, const void *cos,
                            const void *sin, const void *position, int32_t max_seq) {
  return attn_common(q, k, v, out, valid_len, ws, n_q, n_kv, hd, n_split, scale, stream, k_act,
                     v_act, cos, sin, position, max_seq, 0, 1);
}

extern "C" int chr_dv2_attn(const void *q, const void *k, const void *v, void *out,
                            const void *valid_len, int32_t n_q, int32_t n_kv, int32_t hd,
                            int32_t n_waves, float scale, void *stream, const void *k_act,
                            const void *v_act, const void *cos, const void *sin,
                            const void *position, int32_t max_seq) {
  return attn_common(q, k, v, out, valid_len, nullptr, n_q, n_kv, hd, n_waves, scale, stream,
                     k_act, v_act, cos, sin, position, max_seq, 1, 1);
}

extern "C" int64_t chr_dv2_attn_state_floats(int32_t n_q, int32_t hd, int32_t n_parts) {
  if (n_q < 1 || hd < 1 || n_parts < 1) {
    return 0;
  }
  return static_cast<int64_t>(n_q) * n_parts * (hd + 4);
}

extern "C" int chr_dv2_attn_parts(const void *q, const void *k, const void *v,
                                  const void *valid_len, float *state, int32_t n_q, int32_t n_kv,
                                  int32_t hd, int32_t n_parts, int32_t n_waves, float scale,
                                  void *stream, const void *k_act, const void *v_act,
                                  const void *cos, const void *sin, const void *position,
                                  int32_t max_seq) {
  return attn_common(q, k, v, nullptr, valid_len, state, n_q, n_kv, hd, n_waves, scale, stream,
                     k_act, v_act, cos, sin, position, max_seq, 2, n_parts);
}

extern "C" int chr_dv2_attn_chunk(const void *q, const void *k, const void *v, void *out,
                                  const void *first_len, int32_t n_tok, int32_t n_q, int32_t n_kv,
                                  int32_t hd, int32_t n_waves, float scale, void *stream,
                                  int32_t max_seq, int32_t out_tok_stride,
                                  int32_t out_dim_stride) {
  if (out_dim_stride < 1 || out_tok_stride < 0) {
    return -3;
  }
  return attn_common(q, k, v, out, first_len, nullptr, n_q, n_kv, hd, n_waves, scale, stream,
                     nullptr, nullptr, nullptr, nullptr, nullptr, max_seq, 1, 1, n_tok,
                     out_tok_stride, out_dim_stride);
}
