// Measurement program for the fixed cost of a launch on gfx950 (MI355X); no library code, no
// torch.  Six tables, printed as text:
//
//   floor   an empty kernel replayed from a HIP graph of serial nodes, per grid, workgroup size
//           and dynamic LDS size; and the same with one dependent word handed from launch to
//           launch (what a chain of GEMVs pays before its first useful instruction)
//   stream  a pure streaming read of one GEMV's weight bytes (no x, no table, no arithmetic)
//           per grid form and request depth: the ceiling for one cold launch of that size
//   chain   a chain of GEMV-shaped launches (level table in LDS, x staged in LDS, rows streamed
//           and looked up, one output per row), each consuming what the one before wrote:
//           serial graph nodes against launches that alternate between two queues and hand over
//           through device words, so that launch i+1 is resident, has filled its table and has
//           its first weight requests in flight while launch i still streams
//
//   ramp    clock stamps inside a GEMV-shaped launch: where the time before its first product goes
//
//   latency dependent loads of one lane, stamped: what a trip to memory costs at the start of a launch
//
//   code    what straight-line code costs the first time a launch runs through it
//
// Usage: launch_probe [floor] [stream] [chain] [ramp] [latency] [code]   (default: all six)
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CK(x)                                                                              \
  do {                                                                                     \
    hipError_t e_ = (x);                                                                   \
    if (e_ != hipSuccess) {                                                                \
      std::printf("HIP error %s at line %d: %s\n", hipGetErrorString(e_), __LINE__, #x);   \
      std::fflush(stdout);                                                                 \
      std::exit(1);                                                                        \
    }                                                                                      \
  } while (0)

namespace {

typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((ext_vector_type(2))) __bf16 Bf16x2;

constexpr int kCUs = 256;

// ---- timing --------------------------------------------------------------------------
// Median over `reps` replays of a graph, in microseconds per node.
double time_graph(hipGraphExec_t exec, hipStream_t st, int nodes, int reps,
                  void (*before)(hipStream_t, void *) = nullptr, void *ctx = nullptr) {
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  std::vector<float> ms;
  for (int r = 0; r < reps + 1; ++r) {
    if (before != nullptr) {
      before(st, ctx);
    }
    CK(hipEventRecord(e0, st));
    CK(hipGraphLaunch(exec, st));
    CK(hipEventRecord(e1, st));
    CK(hipStreamSynchronize(st));
    float t = 0.f;
    CK(hipEventElapsedTime(&t, e0, e1));
    if (r > 0) {
      ms.push_back(t);
    }
  }
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
  std::sort(ms.begin(), ms.end());
  return ms[ms.size() / 2] * 1e3 / nodes;
}

// ---- floor ---------------------------------------------------------------------------
__global__ void empty_kernel(uint32_t *sink) {
  extern __shared__ uint32_t lds[];
  if (sink == reinterpret_cast<uint32_t *>(1)) {  // never true: keeps the LDS declaration alive
    sink[0] = lds[threadIdx.x];
  }
}

// Thread 0 of every workgroup reads the word the launch before wrote and writes its own.
__global__ void handover_kernel(const uint32_t *in, uint32_t *out) {
  extern __shared__ uint32_t lds[];
  if (threadIdx.x == 0) {
    out[blockIdx.x] = in[blockIdx.x] + 1u;
  }
}

void run_floor(hipStream_t st) {
  std::printf("== floor: microseconds per node, graph of 200 serial kernel nodes, median of 5 replays\n");
  std::printf("%-6s %-8s %-8s %10s %12s\n", "grid", "threads", "lds_KB", "empty", "handover");
  uint32_t *a = nullptr, *b = nullptr;
  CK(hipMalloc(&a, 4096 * 4));
  CK(hipMalloc(&b, 4096 * 4));
  CK(hipMemset(a, 0, 4096 * 4));
  CK(hipMemset(b, 0, 4096 * 4));
  CK(hipFuncSetAttribute(reinterpret_cast<const void *>(empty_kernel),
                         hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024));
  CK(hipFuncSetAttribute(reinterpret_cast<const void *>(handover_kernel),
                         hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024));
  const int nodes = 200;
  for (int grid : {256, 512, 1024}) {
    for (int threads : {256, 512, 1024}) {
      for (int lds_kb : {0, 32, 75}) {
        double us[2];
        for (int kind = 0; kind < 2; ++kind) {
          hipGraph_t g;
          CK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
          for (int i = 0; i < nodes; ++i) {
            if (kind == 0) {
              empty_kernel<<<grid, threads, lds_kb * 1024, st>>>(a);
            } else {
              handover_kernel<<<grid, threads, lds_kb * 1024, st>>>(i % 2 ? a : b, i % 2 ? b : a);
            }
          }
          CK(hipStreamEndCapture(st, &g));
          hipGraphExec_t exec;
          CK(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
          us[kind] = time_graph(exec, st, nodes, 5);
          CK(hipGraphExecDestroy(exec));
          CK(hipGraphDestroy(g));
        }
        std::printf("%-6d %-8d %-8d %10.2f %12.2f\n", grid, threads, lds_kb, us[0], us[1]);
        std::fflush(stdout);
      }
    }
  }
  CK(hipFree(a));
  CK(hipFree(b));
}

// ---- stream --------------------------------------------------------------------------
// Wavefront g of W reads 64*VEC-byte chunks g, g + W, ..; DEPTH requests are issued before the
// first is consumed.
template <int VEC, int DEPTH>
__global__ void stream_read(const uint8_t *w, int chunks, uint32_t *out) {
  const int lane = threadIdx.x & 63;
  const int waves_per_wg = blockDim.x >> 6;
  const int g = blockIdx.x * waves_per_wg + (threadIdx.x >> 6);
  const int W = gridDim.x * waves_per_wg;
  uint32_t acc = 0;
  for (int c = g; c < chunks; c += W * DEPTH) {
    if constexpr (VEC == 8) {
      U32x2 v[DEPTH];
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int cc = min(c + d * W, chunks - 1);
        v[d] = __builtin_nontemporal_load(reinterpret_cast<const U32x2 *>(w) + static_cast<size_t>(cc) * 64 + lane);
      }
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        acc ^= v[d].x ^ v[d].y;
      }
    } else {
      U32x4 v[DEPTH];
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int cc = min(c + d * W, chunks - 1);
        v[d] = __builtin_nontemporal_load(reinterpret_cast<const U32x4 *>(w) + static_cast<size_t>(cc) * 64 + lane);
      }
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        acc ^= v[d].x ^ v[d].y ^ v[d].z ^ v[d].w;
      }
    }
  }
  if (acc == 0x12345678u) {
    out[g] = acc;
  }
}

struct StreamCase {
  const char *name;
  void (*kern)(const uint8_t *, int, uint32_t *);
  int vec;
};

void run_stream(hipStream_t st, const uint8_t *weights, size_t copy_bytes, int copies, uint32_t *out) {
  std::printf("== stream: pure streaming read of %zu bytes per launch (rotating through %d copies), "
              "graph of 48 serial nodes, median of 5 replays\n", copy_bytes, copies);
  std::printf("%-6s %-8s %-22s %10s %10s %8s\n", "grid", "threads", "requests", "us", "TB/s", "of_8");
  const StreamCase cases[] = {
      {"8 B x 2 in flight", stream_read<8, 2>, 8},   {"8 B x 4 in flight", stream_read<8, 4>, 8},
      {"8 B x 8 in flight", stream_read<8, 8>, 8},   {"16 B x 2 in flight", stream_read<16, 2>, 16},
      {"16 B x 4 in flight", stream_read<16, 4>, 16},
  };
  const int nodes = 48;
  const int forms[][2] = {{256, 1024}, {512, 512}, {1024, 256}, {2048, 256}, {4096, 256}};
  for (const auto &f : forms) {
    for (const StreamCase &c : cases) {
      const int chunks = static_cast<int>(copy_bytes / (64 * c.vec));
      hipGraph_t g;
      CK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
      for (int i = 0; i < nodes; ++i) {
        c.kern<<<f[0], f[1], 0, st>>>(weights + static_cast<size_t>(i % copies) * copy_bytes, chunks, out);
      }
      CK(hipStreamEndCapture(st, &g));
      hipGraphExec_t exec;
      CK(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
      const double us = time_graph(exec, st, nodes, 5);
      CK(hipGraphExecDestroy(exec));
      CK(hipGraphDestroy(g));
      const double tbs = copy_bytes / us * 1e-6;
      std::printf("%-6d %-8d %-22s %10.2f %10.2f %8.3f\n", f[0], f[1], c.name, us, tbs, tbs / 8.0);
      std::fflush(stdout);
    }
  }
}

// ---- chain ---------------------------------------------------------------------------
constexpr int kChainThreads = 512;           // half a compute unit: two launches fit side by side
constexpr int kChainWaves = kChainThreads / 64;
constexpr int kTableBytes = 64 * 1024;       // 256 byte values x 64 lane copies x 4 bytes
constexpr int kXBytesMax = 10 * 1024;        // activations of one row
constexpr int kChainLds = kTableBytes + kXBytesMax + 256;
constexpr int kHalfSteps = 5;                // a row is 5 x 512 bytes (K = 5120)

struct ChainArgs {
  const uint8_t *w;    // rows x 2560 bytes
  int rows;
  const uint16_t *x_in;  // what the launch before wrote (bf16), x_bytes of it are read
  uint16_t *y_out;       // one bf16 per row
  int x_bytes;
  // hand-over: mode 0 none (the graph edge orders the launches), 1 one counter that every
  // workgroup of the producer bumps, 2 one word per producer workgroup
  int mode;
  unsigned int *flags;
  unsigned int wait_for;   // counter value / flag value that says "the launch before is done"
  unsigned int signal;     // mode 2: the value this launch leaves in its words
  unsigned int *gave_up;   // set when a bounded wait expired
  long long spin_clocks;   // bound of the wait, 100 MHz clocks
  // read-ahead inside the launch: the weights of the launch after this one; every wavefront
  // touches one dword per 128-byte line of the first `ahead_rows` rows that the same wavefront of
  // the same workgroup will request first there (null: none)
  const uint8_t *next_w;
  int ahead_rows;
};

__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(Bf16x2, a), __builtin_bit_cast(Bf16x2, b), acc, false);
}

__device__ __forceinline__ uint32_t lds_u32(uint32_t addr) {
  return *reinterpret_cast<const __attribute__((address_space(3))) uint32_t *>(addr);
}

__device__ __forceinline__ float row_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    v += __shfl_xor(v, o, 64);
  }
  return v;
}

__global__ __launch_bounds__(kChainThreads, 4) void chain_kernel(const ChainArgs a) {
  extern __shared__ uint4 dyn[];
  uint32_t *table = reinterpret_cast<uint32_t *>(dyn);          // LDS address 0
  uint4 *xs = reinterpret_cast<uint4 *>(reinterpret_cast<char *>(dyn) + kTableBytes);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int grid = gridDim.x;
  const int first = wave * grid + static_cast<int>(blockIdx.x);
  const int stride = grid * kChainWaves;

  // first row's requests: nothing of this depends on the launch before
  U32x2 cur[kHalfSteps], nxt[kHalfSteps];
  {
    const int r = max(min(first, a.rows - 1), 0);
    const U32x2 *p = reinterpret_cast<const U32x2 *>(a.w + static_cast<size_t>(r) * (kHalfSteps * 512)) + lane;
#pragma unroll
    for (int t = 0; t < kHalfSteps; ++t) {
      cur[t] = __builtin_nontemporal_load(p + t * 64);
    }
  }
  uint32_t ahead = 0;
  if (a.next_w != nullptr) {
    // 20 lines of 128 bytes per row; lane l takes line l % 20 of row l / 20 of its first rows
    const int k = lane / 20, line = lane % 20;
    const int r = max(min(first + k * stride, a.rows - 1), 0);  // (rows == 0: row 0 of the copy, which exists)
    if (k < a.ahead_rows && a.rows > 0) {
      ahead = *reinterpret_cast<const uint32_t *>(a.next_w + static_cast<size_t>(r) * (kHalfSteps * 512) + line * 128);
    }
  }
  // the level table: 32 byte values per wavefront, one lane copy each
#pragma unroll
  for (int j = 0; j < 32; ++j) {
    const uint32_t byte = static_cast<uint32_t>(wave) * 32u + j;
    table[(byte << 6) + lane] = (0x3C00u + (byte & 15u)) | ((0x3C00u + (byte >> 4)) << 16);
  }
  // wait for the launch before (bounded: on expiry the launch says so and goes on)
  if (a.mode == 1) {
    if (threadIdx.x == 0) {
      const long long t0 = wall_clock64();
      while (true) {
        const unsigned int v = __hip_atomic_load(a.flags, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (static_cast<int>(v - a.wait_for) >= 0) {
          break;
        }
        if (wall_clock64() - t0 > a.spin_clocks) {
          __hip_atomic_store(a.gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
    }
  } else if (a.mode == 2) {
    if (wave == 0) {
      const long long t0 = wall_clock64();
      while (true) {
        bool ok = true;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int i = min(lane + 64 * j, grid - 1);
          const unsigned int v = __hip_atomic_load(a.flags + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          ok = ok && static_cast<int>(v - a.wait_for) >= 0;
        }
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
          break;
        }
        if (wall_clock64() - t0 > a.spin_clocks) {
          if (lane == 0) {
            __hip_atomic_store(a.gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
    }
  }
  __syncthreads();
  // x: written by other compute dies a moment ago when the launches overlap, so it is read
  // past the caches then
  {
    const int nvec = a.x_bytes >> 4;
    for (int i = threadIdx.x; i < nvec; i += kChainThreads) {
      uint4 v;
      if (a.mode == 0) {
        v = reinterpret_cast<const uint4 *>(a.x_in)[i];
      } else {
        const unsigned long long *p = reinterpret_cast<const unsigned long long *>(a.x_in) + 2 * i;
        const unsigned long long lo = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long hi = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        v = make_uint4(static_cast<uint32_t>(lo), static_cast<uint32_t>(lo >> 32), static_cast<uint32_t>(hi),
                       static_cast<uint32_t>(hi >> 32));
      }
      // keep the numbers tame whatever the bytes are: exponent of 2^-7
      v.x = (v.x & 0x007F007Fu) | 0x3C003C00u;
      v.y = (v.y & 0x007F007Fu) | 0x3C003C00u;
      v.z = (v.z & 0x007F007Fu) | 0x3C003C00u;
      v.w = (v.w & 0x007F007Fu) | 0x3C003C00u;
      xs[i] = v;
    }
  }
  __syncthreads();

  const uint32_t lane4 = static_cast<uint32_t>(lane) << 2;
  for (int row = first; row < a.rows; row += stride) {
    const int rn = min(row + stride, a.rows - 1);
    const U32x2 *p = reinterpret_cast<const U32x2 *>(a.w + static_cast<size_t>(rn) * (kHalfSteps * 512)) + lane;
#pragma unroll
    for (int t = 0; t < kHalfSteps; ++t) {
      nxt[t] = __builtin_nontemporal_load(p + t * 64);
    }
    float acc = 0.f;
#pragma unroll
    for (int t = 0; t < kHalfSteps; ++t) {
      const uint4 x0 = xs[t * 128 + lane];
      const uint4 x1 = xs[t * 128 + 64 + lane];
      const uint32_t wx = cur[t].x, wy = cur[t].y;
      float pa = 0.f, pb = 0.f;
      pa = dot2(lds_u32(__builtin_amdgcn_perm(wx, lane4, 0x0C0C0400u)), x0.x, pa);
      pb = dot2(lds_u32(__builtin_amdgcn_perm(wx, lane4, 0x0C0C0500u)), x0.y, pb);
      pa = dot2(lds_u32(__builtin_amdgcn_perm(wx, lane4, 0x0C0C0600u)), x0.z, pa);
      pb = dot2(lds_u32(__builtin_amdgcn_perm(wx, lane4, 0x0C0C0700u)), x0.w, pb);
      pa = dot2(lds_u32(__builtin_amdgcn_perm(wy, lane4, 0x0C0C0400u)), x1.x, pa);
      pb = dot2(lds_u32(__builtin_amdgcn_perm(wy, lane4, 0x0C0C0500u)), x1.y, pb);
      pa = dot2(lds_u32(__builtin_amdgcn_perm(wy, lane4, 0x0C0C0600u)), x1.z, pa);
      pb = dot2(lds_u32(__builtin_amdgcn_perm(wy, lane4, 0x0C0C0700u)), x1.w, pb);
      acc += pa + pb;
    }
    acc = row_sum(acc);
    if (lane == 0) {
      const uint16_t o = static_cast<uint16_t>(__float_as_uint(acc) >> 16);
      if (a.mode == 0) {
        a.y_out[row] = o;
      } else {
        __hip_atomic_store(a.y_out + row, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
#pragma unroll
    for (int t = 0; t < kHalfSteps; ++t) {
      cur[t] = nxt[t];
    }
  }
  asm volatile("" ::"v"(ahead));
  if (a.mode != 0) {
    // every store of this workgroup has reached memory before the workgroup says it is done
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
      if (a.mode == 1) {
        __hip_atomic_fetch_add(a.flags, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        __hip_atomic_store(a.flags + blockIdx.x, a.signal, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}


// What the workgroups of a chain launch will request first, read ahead of time by a small launch
// that runs beside the chain launch before it: workgroup b touches the first `depth` rows of every
// wavefront of workgroup b of the launch it reads for, so that they wait in that compute die's L2.
__global__ __launch_bounds__(256) void prefetch_kernel(const uint8_t *w, int rows, int consumer_waves, int depth,
                                                       uint32_t *sink) {
  const int grid = gridDim.x;
  const int b = blockIdx.x;
  const int chunks = consumer_waves * depth * (kHalfSteps * 32);  // 16-byte chunks of this workgroup
  uint32_t acc = 0;
  for (int c0 = threadIdx.x; c0 < chunks; c0 += 4 * 256) {
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = min(c0 + u * 256, chunks - 1);
      const int slot = c / (kHalfSteps * 32), off = c % (kHalfSteps * 32);
      const int cw = slot % consumer_waves, pass = slot / consumer_waves;
      const int row = min(cw * grid + b + pass * grid * consumer_waves, rows - 1);
      v[u] = reinterpret_cast<const uint4 *>(w + static_cast<size_t>(row) * (kHalfSteps * 512))[off];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
  }
  if (acc == 0x12345678u) {
    sink[b] = acc;
  }
}

struct ChainCtx {
  unsigned int *flags;
};

void reset_flags(hipStream_t st, void *ctx) {
  CK(hipMemsetAsync(static_cast<ChainCtx *>(ctx)->flags, 0, 4096, st));
}

// topology 0: serial nodes, hand-over by the graph edge (mode 0)
// topology 1: node i depends on node i-2 only (two queues), hand-over by device words (mode 1 / 2)
// topology 2: serial nodes, but the kernels still signal and wait through device words (what the
//             hand-over code itself costs when nothing overlaps)
// topology 3 / 4: serial nodes, and beside node i-1 a small node that reads the first 1 / 2 rows of
//             every wavefront of node i ahead of time (it follows node i-2 and nothing follows it)
// topology 5 / 6 / 7: serial nodes; every wavefront of node i touches the lines of the first 1 / 2 / 3
//             rows that its counterpart in node i+1 will request first
double run_chain_case(hipStream_t st, const uint8_t *weights, size_t copy_bytes, int copies, int rows,
                      int topology, int mode, uint16_t *ya, uint16_t *yb, unsigned int *flags,
                      unsigned int *gave_up, int nodes, long long spin_clocks) {
  hipGraph_t g;
  CK(hipGraphCreate(&g, 0));
  std::vector<hipGraphNode_t> node(nodes);
  std::vector<ChainArgs> args(nodes);
  for (int i = 0; i < nodes; ++i) {
    ChainArgs &a = args[i];
    a.w = weights + static_cast<size_t>(i % copies) * copy_bytes;
    a.rows = rows;
    a.x_in = i % 2 ? ya : yb;
    a.y_out = i % 2 ? yb : ya;
    a.x_bytes = kXBytesMax;
    a.mode = mode;
    a.flags = flags;
    a.gave_up = gave_up;
    a.spin_clocks = spin_clocks;
    a.next_w = topology >= 5 && rows > 0 ? weights + static_cast<size_t>((i + 1) % copies) * copy_bytes : nullptr;
    a.ahead_rows = topology - 4;
    if (mode == 1) {
      a.wait_for = static_cast<unsigned int>(i) * kCUs;  // i launches before this one, kCUs bumps each
      a.signal = 0;
    } else {
      a.wait_for = static_cast<unsigned int>(i);  // the launch before left i (launch 0 waits for 0)
      a.signal = static_cast<unsigned int>(i) + 1u;
    }
    void *params[] = {&a};
    hipKernelNodeParams kp{};
    kp.func = reinterpret_cast<void *>(chain_kernel);
    kp.gridDim = dim3(kCUs);
    kp.blockDim = dim3(kChainThreads);
    kp.sharedMemBytes = kChainLds;
    kp.kernelParams = params;
    kp.extra = nullptr;
    std::vector<hipGraphNode_t> deps;
    if (topology == 1) {
      if (i >= 2) {
        deps.push_back(node[i - 2]);
      }
    } else if (i >= 1) {
      deps.push_back(node[i - 1]);
    }
    CK(hipGraphAddKernelNode(&node[i], g, deps.data(), deps.size(), &kp));
    if ((topology == 3 || topology == 4) && rows > 0) {
      const uint8_t *pw = a.w;
      int prows = rows, cwaves = kChainWaves, depth = topology - 2;
      uint32_t *sink = reinterpret_cast<uint32_t *>(flags);
      void *pparams[] = {&pw, &prows, &cwaves, &depth, &sink};
      hipKernelNodeParams pp{};
      pp.func = reinterpret_cast<void *>(prefetch_kernel);
      pp.gridDim = dim3(kCUs);
      pp.blockDim = dim3(256);
      pp.sharedMemBytes = 0;
      pp.kernelParams = pparams;
      pp.extra = nullptr;
      std::vector<hipGraphNode_t> pdeps;
      if (i >= 2) {
        pdeps.push_back(node[i - 2]);
      }
      hipGraphNode_t pn;
      CK(hipGraphAddKernelNode(&pn, g, pdeps.data(), pdeps.size(), &pp));
    }
  }
  hipGraphExec_t exec;
  CK(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
  ChainCtx ctx{flags};
  const double us = time_graph(exec, st, nodes, 5, reset_flags, &ctx);
  CK(hipGraphExecDestroy(exec));
  CK(hipGraphDestroy(g));
  return us;
}

void run_chain(hipStream_t st, const uint8_t *weights, size_t copy_bytes, int copies) {
  CK(hipFuncSetAttribute(reinterpret_cast<const void *>(chain_kernel),
                         hipFuncAttributeMaxDynamicSharedMemorySize, kChainLds));
  int per_cu = 0;
  CK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, chain_kernel, kChainThreads, kChainLds));
  std::printf("== chain: GEMV-shaped launches of %d threads x %d workgroups, %d B of LDS, "
              "%d workgroups fit a compute unit\n", kChainThreads, kCUs, kChainLds, per_cu);
  uint16_t *ya = nullptr, *yb = nullptr;
  unsigned int *flags = nullptr, *gave_up = nullptr;
  CK(hipMalloc(&ya, 64 * 1024));
  CK(hipMalloc(&yb, 64 * 1024));
  CK(hipMalloc(&flags, 4096));
  CK(hipMalloc(&gave_up, 256));
  CK(hipMemset(ya, 0, 64 * 1024));
  CK(hipMemset(yb, 0, 64 * 1024));
  CK(hipMemset(gave_up, 0, 256));
  const int nodes = 200;
  const long long spin = 2'000'000;  // 20 ms of the 100 MHz clock
  std::printf("%-10s %-38s %-26s %10s %10s\n", "rows", "topology", "hand-over", "us/launch", "gave_up");
  if (per_cu < 2) {
    std::printf("two launches do not fit a compute unit side by side: overlapped cases skipped\n");
  }
  const int max_rows = static_cast<int>(copy_bytes / (kHalfSteps * 512));
  for (int rows : {0, 5120, 7168, 13824}) {
    if (rows > max_rows) {
      continue;
    }
    struct Case {
      int topology, mode;
      const char *tname, *hname;
    };
    const Case cases[] = {
        {0, 0, "serial nodes", "graph edge"},
        {2, 1, "serial nodes", "edge + one counter"},
        {2, 2, "serial nodes", "edge + word per workgroup"},
        {1, 1, "node i after node i-2 (two queues)", "one counter"},
        {1, 2, "node i after node i-2 (two queues)", "word per workgroup"},
        {3, 0, "serial + read-ahead node, 1 row/wave", "graph edge"},
        {5, 0, "serial, launch reads 1 row/wave ahead", "graph edge"},
        {6, 0, "serial, launch reads 2 rows/wave ahead", "graph edge"},
        {7, 0, "serial, launch reads 3 rows/wave ahead", "graph edge"},
    };
    for (const Case &c : cases) {
      if (c.topology == 1 && per_cu < 2) {
        continue;
      }
      CK(hipMemset(gave_up, 0, 256));
      const double us = run_chain_case(st, weights, copy_bytes, copies, rows, c.topology, c.mode, ya, yb, flags,
                                       gave_up, nodes, spin);
      unsigned int gu = 0;
      CK(hipMemcpy(&gu, gave_up, 4, hipMemcpyDeviceToHost));
      std::printf("%-10d %-38s %-26s %10.2f %10u\n", rows, c.tname, c.hname, us, gu);
      std::fflush(stdout);
      if (gu != 0) {
        std::printf("a bounded wait expired: the remaining overlapped cases of this size are skipped\n");
        break;
      }
    }
  }
  // the bounded wait itself: a consumer whose producer is never launched gives up and exits
  {
    CK(hipMemset(flags, 0, 4096));
    CK(hipMemset(gave_up, 0, 256));
    ChainArgs a{};
    a.w = weights;
    a.rows = 256;
    a.x_in = ya;
    a.y_out = yb;
    a.x_bytes = kXBytesMax;
    a.mode = 2;
    a.flags = flags;
    a.wait_for = 7;  // nobody ever writes 7
    a.signal = 8;
    a.gave_up = gave_up;
    a.spin_clocks = 20'000;  // 0.2 ms
    chain_kernel<<<kCUs, kChainThreads, kChainLds, st>>>(a);
    CK(hipStreamSynchronize(st));
    unsigned int gu = 0;
    CK(hipMemcpy(&gu, gave_up, 4, hipMemcpyDeviceToHost));
    std::printf("bounded wait with no producer launched: gave_up = %u (1 expected), kernel returned\n", gu);
  }
  CK(hipFree(ya));
  CK(hipFree(yb));
  CK(hipFree(flags));
  CK(hipFree(gave_up));
}

// ---- ramp ----------------------------------------------------------------------------
// Where the time before a GEMV's first product goes: every wavefront of a launch stamps the
// 100 MHz clock (one counter for the whole device) at its first instruction, when its kernel
// arguments have arrived, when x has arrived, when x is usable (after the LDS copy and the
// workgroup's barrier, or at once when every wavefront reads x into registers itself), when its
// first row of weights has arrived, and at its end.  Launches are serial graph nodes; the gap
// is the earliest entry of a launch minus the latest end of the one before.
constexpr int kStamps = 6;

struct RampArgs {
  const uint8_t *w;
  const uint16_t *x;
  uint16_t *y;
  long long *stamps;  // [wavefront][kStamps]
  int rows;
  int x_mode;   // 0: every thread copies one or two pieces of x to LDS; 1: every wavefront reads x into
                // registers itself; 2: the workgroup's first wavefront copies all of x to LDS
  int w_first;  // half steps of weights requested before x is waited for (the rest right after)
  int table;    // level table: 0 one dword store per entry before x is waited for, 1 the same after x
                // has arrived, 2 four entries per 16-byte store before, 3 not filled at all
};

// x was requested before the first w_first half steps of weights: it has arrived when at most
// those are outstanding
__device__ __forceinline__ void wait_all_but(int younger) {
  if (younger >= 5) {
    asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
  } else if (younger >= 1) {
    asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
}

template <bool SCALAR_ARGS>
__device__ __forceinline__ void ramp_body(const uint8_t *w, const uint16_t *x, uint16_t *y, long long *stamps,
                                          int rows, int x_mode, int w_first, int table_mode, long long t_entry) {
  const bool direct_x = x_mode == 1;
  extern __shared__ uint4 dyn[];
  uint32_t *table = reinterpret_cast<uint32_t *>(dyn);
  uint4 *xs = reinterpret_cast<uint4 *>(reinterpret_cast<char *>(dyn) + kTableBytes);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int waves = blockDim.x >> 6;
  const int gw = static_cast<int>(blockIdx.x) * waves + wave;
  // the first use of an argument: its value has arrived when this statement is passed
  asm volatile("; uses %0" ::"s"(x));
  const long long t_args = wall_clock64();
  const int first = wave * static_cast<int>(gridDim.x) + static_cast<int>(blockIdx.x);
  const int r = max(min(first, rows - 1), 0);
  uint4 xv[10];
  uint4 xl0 = make_uint4(0, 0, 0, 0), xl1 = xl0;
  if (direct_x) {
    // lane l of half step t multiplies x[1024 t + 16 l .. + 16): two 16-byte pieces
#pragma unroll
    for (int t = 0; t < kHalfSteps; ++t) {
      xv[2 * t] = reinterpret_cast<const uint4 *>(x)[t * 128 + 2 * lane];
      xv[2 * t + 1] = reinterpret_cast<const uint4 *>(x)[t * 128 + 2 * lane + 1];
    }
  } else if (x_mode == 2) {
    if (wave == 0) {
#pragma unroll
      for (int j = 0; j < 10; ++j) {
        xv[j] = reinterpret_cast<const uint4 *>(x)[j * 64 + lane];
      }
    }
  } else {
    // 640 pieces of 16 bytes, two per thread of a 512-thread workgroup (one of a 1024-thread one)
    const int i0 = min(static_cast<int>(threadIdx.x), 639);
    const int i1 = min(static_cast<int>(threadIdx.x + blockDim.x), 639);
    xl0 = reinterpret_cast<const uint4 *>(x)[i0];
    xl1 = reinterpret_cast<const uint4 *>(x)[i1];
  }
  U32x2 cur[kHalfSteps];
  const U32x2 *p = reinterpret_cast<const U32x2 *>(w + static_cast<size_t>(r) * (kHalfSteps * 512)) + lane;
#pragma unroll
  for (int t = 0; t < kHalfSteps; ++t) {
    cur[t] = U32x2{0u, 0u};
    if (t < w_first) {
      cur[t] = __builtin_nontemporal_load(p + t * 64);
    }
  }
  const int per_wave = 256 / waves;
  auto fill_table = [&]() {
    if (table_mode == 2) {
      // a byte's 64 lane copies are 256 contiguous bytes of one value: lane l writes 16 bytes of the
      // row of byte 4 j + l / 16
      for (int j = 0; j < per_wave / 4; ++j) {
        const uint32_t byte = static_cast<uint32_t>(wave * per_wave + 4 * j + (lane >> 4));
        const uint32_t v = (0x3C00u + (byte & 15u)) | ((0x3C00u + (byte >> 4)) << 16);
        reinterpret_cast<uint4 *>(table)[(byte << 4) + (lane & 15)] = make_uint4(v, v, v, v);
      }
    } else if (table_mode != 3) {
#pragma unroll 4
      for (int j = 0; j < per_wave; ++j) {
        const uint32_t byte = static_cast<uint32_t>(wave * per_wave + j);
        table[(byte << 6) + lane] = (0x3C00u + (byte & 15u)) | ((0x3C00u + (byte >> 4)) << 16);
      }
    }
  };
  if (table_mode != 1) {
    fill_table();
  }
  long long t_x, t_usable;
  if (direct_x) {
    wait_all_but(w_first);
#pragma unroll
    for (int i = 0; i < 10; ++i) {
      asm volatile("" : "+v"(xv[i].x), "+v"(xv[i].y), "+v"(xv[i].z), "+v"(xv[i].w));
    }
    t_x = wall_clock64();
    if (table_mode == 1) {
      fill_table();
    }
    __syncthreads();  // the table
    t_usable = wall_clock64();
  } else {
    if (x_mode == 2) {
      if (wave == 0) {
        wait_all_but(w_first);
#pragma unroll
        for (int j = 0; j < 10; ++j) {
          asm volatile("" : "+v"(xv[j].x), "+v"(xv[j].y), "+v"(xv[j].z), "+v"(xv[j].w));
          xs[j * 64 + lane] = xv[j];
        }
      }
      t_x = wall_clock64();
    } else {
      wait_all_but(w_first);
      asm volatile("" : "+v"(xl0.x), "+v"(xl1.x));
      t_x = wall_clock64();
      xs[min(static_cast<int>(threadIdx.x), 639)] = xl0;
      if (threadIdx.x + blockDim.x < 640) {
        xs[threadIdx.x + blockDim.x] = xl1;
      }
    }
    if (table_mode == 1) {
      fill_table();
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < kHalfSteps; ++t) {
      xv[2 * t] = xs[t * 128 + lane];
      xv[2 * t + 1] = xs[t * 128 + 64 + lane];
    }
#pragma unroll
    for (int i = 0; i < 10; ++i) {
      asm volatile("" : "+v"(xv[i].x), "+v"(xv[i].y), "+v"(xv[i].z), "+v"(xv[i].w));
    }
    t_usable = wall_clock64();
  }
#pragma unroll
  for (int t = 0; t < kHalfSteps; ++t) {
    if (t >= w_first) {
      cur[t] = __builtin_nontemporal_load(p + t * 64);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int t = 0; t < kHalfSteps; ++t) {
    asm volatile("" : "+v"(cur[t].x), "+v"(cur[t].y));
  }
  const long long t_w = wall_clock64();
  // one row, so that the launch does what a GEMV's first row does
  const uint32_t lane4 = static_cast<uint32_t>(lane) << 2;
  float acc = 0.f;
#pragma unroll
  for (int t = 0; t < kHalfSteps; ++t) {
    const uint4 x0 = xv[2 * t], x1 = xv[2 * t + 1];
    const uint32_t wx = cur[t].x, wy = cur[t].y;
    float pa = 0.f, pb = 0.f;
    pa = dot2(lds_u32(__builtin_amdgcn_perm(wx, lane4, 0x0C0C0400u)), x0.x, pa);
    pb = dot2(lds_u32(__builtin_amdgcn_perm(wx, lane4, 0x0C0C0500u)), x0.y, pb);
    pa = dot2(lds_u32(__builtin_amdgcn_perm(wx, lane4, 0x0C0C0600u)), x0.z, pa);
    pb = dot2(lds_u32(__builtin_amdgcn_perm(wx, lane4, 0x0C0C0700u)), x0.w, pb);
    pa = dot2(lds_u32(__builtin_amdgcn_perm(wy, lane4, 0x0C0C0400u)), x1.x, pa);
    pb = dot2(lds_u32(__builtin_amdgcn_perm(wy, lane4, 0x0C0C0500u)), x1.y, pb);
    pa = dot2(lds_u32(__builtin_amdgcn_perm(wy, lane4, 0x0C0C0600u)), x1.z, pa);
    pb = dot2(lds_u32(__builtin_amdgcn_perm(wy, lane4, 0x0C0C0700u)), x1.w, pb);
    acc += pa + pb;
  }
  acc = row_sum(acc);
  if (lane == 0 && first < rows) {
    y[first] = static_cast<uint16_t>(__float_as_uint(acc) >> 16);
  }
  const long long t_end = wall_clock64();
  if (lane == 0) {
    long long *s = stamps + static_cast<size_t>(gw) * kStamps;
    s[0] = t_entry;
    s[1] = t_args;
    s[2] = t_x;
    s[3] = t_usable;
    s[4] = t_w;
    s[5] = t_end;
  }
}

__global__ __launch_bounds__(1024) void ramp_struct(const RampArgs a) {
  const long long t_entry = wall_clock64();
  ramp_body<false>(a.w, a.x, a.y, a.stamps, a.rows, a.x_mode, a.w_first, a.table, t_entry);
}

// the same with the arguments as scalars, which the build asks to be placed in registers
// before the wavefront starts (no trip to memory for them)
__global__ __launch_bounds__(1024) void ramp_scalar(const uint8_t *w, const uint16_t *x, uint16_t *y,
                                                    long long *stamps, int rows, int x_mode, int w_first, int table) {
  const long long t_entry = wall_clock64();
  ramp_body<true>(w, x, y, stamps, rows, x_mode, w_first, table, t_entry);
}

void run_ramp(hipStream_t st, const uint8_t *weights, size_t copy_bytes, int copies) {
  CK(hipFuncSetAttribute(reinterpret_cast<const void *>(ramp_struct),
                         hipFuncAttributeMaxDynamicSharedMemorySize, kChainLds));
  CK(hipFuncSetAttribute(reinterpret_cast<const void *>(ramp_scalar),
                         hipFuncAttributeMaxDynamicSharedMemorySize, kChainLds));
  const int nodes = 24;
  const int max_waves = 4096;
  uint16_t *x = nullptr, *y = nullptr;
  long long *stamps = nullptr;
  CK(hipMalloc(&x, 64 * 1024));
  CK(hipMalloc(&y, 64 * 1024));
  CK(hipMemset(x, 0, 64 * 1024));
  CK(hipMalloc(&stamps, static_cast<size_t>(nodes) * max_waves * kStamps * 8));
  std::vector<long long> host(static_cast<size_t>(nodes) * max_waves * kStamps);
  std::printf("== ramp: one row per wavefront, serial graph nodes, clock stamps in microseconds; medians over "
              "wavefronts and launches, entry and later stamps relative to the launch's earliest entry\n");
  std::printf("%-6s %-8s %-8s %-16s | %6s | %6s %6s | %6s %6s %6s %6s | %6s %6s | %8s\n", "grid", "threads", "args",
              "x,first w,table", "gap", "entry", "e.max", "args", "x", "usable", "wts", "end", "e.max", "us/node");
  struct Form {
    int grid, threads;
  };
  static const char *const kXNames[] = {"LDS", "registers", "LDS/wave0"};
  for (const Form f : {Form{256, 1024}, Form{512, 512}, Form{256, 512}}) {
    const int waves = f.grid * f.threads / 64;
    for (int scalar = 0; scalar < 2; ++scalar) {
      for (int xw = 0; xw < 9 + 6; ++xw) {
        // cases 9..14: x through LDS by every thread, table filled after x / with wide stores / not at all
        const int direct = xw < 9 ? xw / 3 : 0;       // x_mode
        const int w_first = xw < 9 ? (xw % 3 == 0 ? 5 : (xw % 3 == 1 ? 1 : 0)) : ((xw - 9) % 2 == 0 ? 5 : 0);
        const int table_mode = xw < 9 ? 0 : 1 + (xw - 9) / 2;
        if (scalar == 1 && !(w_first == 5 && direct == 0 && table_mode == 0)) {
          continue;  // the argument form matters (or not) independently of the rest
        }
        hipGraph_t g;
        CK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        for (int i = 0; i < nodes; ++i) {
          const uint8_t *w = weights + static_cast<size_t>(i % copies) * copy_bytes;
          long long *sp = stamps + static_cast<size_t>(i) * max_waves * kStamps;
          if (scalar) {
            ramp_scalar<<<f.grid, f.threads, kChainLds, st>>>(w, x, y, sp, waves, direct, w_first, table_mode);
          } else {
            RampArgs a{w, x, y, sp, waves, direct, w_first, table_mode};
            ramp_struct<<<f.grid, f.threads, kChainLds, st>>>(a);
          }
        }
        CK(hipStreamEndCapture(st, &g));
        hipGraphExec_t exec;
        CK(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
        const double us = time_graph(exec, st, nodes, 3);
        CK(hipMemcpy(host.data(), stamps, host.size() * 8, hipMemcpyDeviceToHost));
        CK(hipGraphExecDestroy(exec));
        CK(hipGraphDestroy(g));
        // per launch: earliest entry, latest end; medians of the per-wavefront offsets
        std::vector<double> gap, col[kStamps], entry_max, end_max;
        long long prev_end = 0;
        for (int i = 0; i < nodes; ++i) {
          const long long *s = host.data() + static_cast<size_t>(i) * max_waves * kStamps;
          long long e0 = s[0], e1 = s[5];
          for (int wv = 0; wv < waves; ++wv) {
            e0 = std::min(e0, s[wv * kStamps]);
            e1 = std::max(e1, s[wv * kStamps + 5]);
          }
          if (i >= 4) {  // the first launches of a replay start from an idle device
            gap.push_back((e0 - prev_end) * 0.01);
            std::vector<double> v[kStamps];
            for (int wv = 0; wv < waves; ++wv) {
              for (int k = 0; k < kStamps; ++k) {
                v[k].push_back((s[wv * kStamps + k] - e0) * 0.01);
              }
            }
            for (int k = 0; k < kStamps; ++k) {
              std::sort(v[k].begin(), v[k].end());
              col[k].push_back(v[k][v[k].size() / 2]);
            }
            entry_max.push_back(v[0].back());
            end_max.push_back(v[5].back());
          }
          prev_end = e1;
        }
        auto med = [](std::vector<double> &v) {
          std::sort(v.begin(), v.end());
          return v[v.size() / 2];
        };
        char xname[32];
        std::snprintf(xname, sizeof xname, "%s,w%d,t%d", kXNames[direct], w_first, table_mode);
        std::printf("%-6d %-8d %-8s %-16s | %6.2f | %6.2f %6.2f | %6.2f %6.2f %6.2f %6.2f | %6.2f %6.2f | %8.2f\n",
                    f.grid, f.threads, scalar ? "scalar" : "struct", xname, med(gap),
                    med(col[0]), med(entry_max), med(col[1]), med(col[2]), med(col[3]), med(col[4]), med(col[5]),
                    med(end_max), us);
        std::fflush(stdout);
      }
    }
  }
  CK(hipFree(x));
  CK(hipFree(y));
  CK(hipFree(stamps));
}

// ---- latency -------------------------------------------------------------------------
// Dependent loads by one lane per workgroup, stamped: the first load of a launch (a line the
// launch before also read), a line nobody has read for many launches, the same line again, a
// line another workgroup of the launch before wrote.  Serial graph nodes.
__global__ __launch_bounds__(256) void latency_kernel(const uint32_t *quiet, const uint32_t *cold,
                                                      const uint32_t *written, uint32_t *to_write, int node,
                                                      long long *stamps) {
  if (threadIdx.x != 0) {
    return;
  }
  const long long t0 = wall_clock64();
  const uint32_t b = blockIdx.x;
  uint32_t v = __builtin_nontemporal_load(quiet + b * 32);  // read by every launch
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(v)::"memory");
  const long long t1 = wall_clock64();
  // 256 KiB further on for every node: untouched since the buffer was cleared
  const uint32_t *c = cold + (static_cast<size_t>(node) << 16) + b * 32 + (v & 1u);
  uint32_t u = *c;
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(u)::"memory");
  const long long t2 = wall_clock64();
  uint32_t u2 = *reinterpret_cast<const volatile uint32_t *>(c + (u & 1u));
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(u2)::"memory");
  const long long t3 = wall_clock64();
  // what workgroup b + 1 of the launch before wrote (another compute die, as a rule)
  uint32_t w = written[((b + 1) % gridDim.x) * 32 + (u2 & 1u)];
  asm volatile("s_waitcnt vmcnt(0)" : "+v"(w)::"memory");
  const long long t4 = wall_clock64();
  to_write[b * 32] = w + 1u;
  long long *s = stamps + (static_cast<size_t>(node) * gridDim.x + b) * 5;
  s[0] = t0;
  s[1] = t1;
  s[2] = t2;
  s[3] = t3;
  s[4] = t4;
}

void run_latency(hipStream_t st) {
  const int nodes = 40, grid = 256;
  uint32_t *quiet = nullptr, *cold = nullptr, *wa = nullptr, *wb = nullptr;
  long long *stamps = nullptr;
  CK(hipMalloc(&quiet, 64 * 1024));
  CK(hipMalloc(&cold, static_cast<size_t>(nodes + 1) << 18));
  CK(hipMalloc(&wa, 64 * 1024));
  CK(hipMalloc(&wb, 64 * 1024));
  CK(hipMalloc(&stamps, static_cast<size_t>(nodes) * grid * 5 * 8));
  CK(hipMemset(quiet, 0, 64 * 1024));
  CK(hipMemset(cold, 0, static_cast<size_t>(nodes + 1) << 18));
  CK(hipMemset(wa, 0, 64 * 1024));
  CK(hipMemset(wb, 0, 64 * 1024));
  hipGraph_t g;
  CK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
  for (int i = 0; i < nodes; ++i) {
    latency_kernel<<<grid, 256, 0, st>>>(quiet, cold, i % 2 ? wa : wb, i % 2 ? wb : wa, i, stamps);
  }
  CK(hipStreamEndCapture(st, &g));
  hipGraphExec_t exec;
  CK(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
  CK(hipGraphLaunch(exec, st));
  CK(hipStreamSynchronize(st));
  std::vector<long long> h(static_cast<size_t>(nodes) * grid * 5);
  CK(hipMemcpy(h.data(), stamps, h.size() * 8, hipMemcpyDeviceToHost));
  std::vector<double> d[4];
  for (int i = 4; i < nodes; ++i) {
    for (int b = 0; b < grid; ++b) {
      const long long *s = h.data() + (static_cast<size_t>(i) * grid + b) * 5;
      for (int k = 0; k < 4; ++k) {
        d[k].push_back((s[k + 1] - s[k]) * 0.01);
      }
    }
  }
  std::printf("== latency: one lane per workgroup, 256 workgroups, dependent loads, microseconds "
              "(median / 10th / 90th percentile over workgroups and launches)\n");
  const char *names[4] = {"first load of the launch, line read by every launch",
                          "line not read since it was cleared", "the same line again",
                          "line written by another workgroup of the launch before"};
  for (int k = 0; k < 4; ++k) {
    std::sort(d[k].begin(), d[k].end());
    std::printf("  %-58s %6.2f %6.2f %6.2f\n", names[k], d[k][d[k].size() / 2], d[k][d[k].size() / 10],
                d[k][d[k].size() * 9 / 10]);
  }
  CK(hipGraphExecDestroy(exec));
  CK(hipGraphDestroy(g));
  CK(hipFree(quiet));
  CK(hipFree(cold));
  CK(hipFree(wa));
  CK(hipFree(wb));
  CK(hipFree(stamps));
}

// ---- code ----------------------------------------------------------------------------
// What straight-line code costs the first time a launch runs through it: a sled of N four-byte
// instructions, passed twice by one wavefront per workgroup, each pass stamped.  The first pass
// fetches the instructions from wherever a launch finds them at its start, the second finds them
// in the instruction cache.
template <int N>
__device__ __forceinline__ void sled() {
  if constexpr (N >= 64) {
    sled<N / 2>();
    sled<N - N / 2>();
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      asm volatile("s_nop 0");
    }
  }
}

template <int N>
__global__ __launch_bounds__(64) void code_kernel(long long *stamps, int node) {
  long long t[3];
  t[0] = wall_clock64();
#pragma unroll 1
  for (int pass = 0; pass < 2; ++pass) {
    sled<N>();
    t[pass + 1] = wall_clock64();
  }
  if (threadIdx.x == 0) {
    long long *s = stamps + (static_cast<size_t>(node) * gridDim.x + blockIdx.x) * 3;
    s[0] = t[0];
    s[1] = t[1];
    s[2] = t[2];
  }
}

template <int N>
void run_code_case(hipStream_t st, long long *stamps, std::vector<long long> &h) {
  const int nodes = 24, grid = 256;
  hipGraph_t g;
  CK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
  for (int i = 0; i < nodes; ++i) {
    code_kernel<N><<<grid, 64, 0, st>>>(stamps, i);
  }
  CK(hipStreamEndCapture(st, &g));
  hipGraphExec_t exec;
  CK(hipGraphInstantiate(&exec, g, nullptr, nullptr, 0));
  const double us = time_graph(exec, st, nodes, 3);
  CK(hipMemcpy(h.data(), stamps, static_cast<size_t>(nodes) * grid * 3 * 8, hipMemcpyDeviceToHost));
  std::vector<double> first, second;
  for (int i = 4; i < nodes; ++i) {
    for (int b = 0; b < grid; ++b) {
      const long long *s = h.data() + (static_cast<size_t>(i) * grid + b) * 3;
      first.push_back((s[1] - s[0]) * 0.01);
      second.push_back((s[2] - s[1]) * 0.01);
    }
  }
  std::sort(first.begin(), first.end());
  std::sort(second.begin(), second.end());
  std::printf("  %6d instructions (%5.1f KB)  first pass %6.2f  second pass %6.2f  us/node %6.2f\n", N, N * 4 / 1024.0,
              first[first.size() / 2], second[second.size() / 2], us);
  std::fflush(stdout);
  CK(hipGraphExecDestroy(exec));
  CK(hipGraphDestroy(g));
}

void run_code(hipStream_t st) {
  long long *stamps = nullptr;
  CK(hipMalloc(&stamps, 24 * 256 * 3 * 8));
  std::vector<long long> h(24 * 256 * 3);
  std::printf("== code: a sled of s_nop passed twice by one wavefront per workgroup (256 workgroups, serial graph "
              "nodes), microseconds per pass, median\n");
  run_code_case<64>(st, stamps, h);
  run_code_case<256>(st, stamps, h);
  run_code_case<512>(st, stamps, h);
  run_code_case<1024>(st, stamps, h);
  run_code_case<2048>(st, stamps, h);
  run_code_case<4096>(st, stamps, h);
  CK(hipFree(stamps));
}

}  // namespace

int main(int argc, char **argv) {
  bool floor = argc == 1, stream = argc == 1, chain = argc == 1, ramp = argc == 1, latency = argc == 1, code = argc == 1;
  for (int i = 1; i < argc; ++i) {
    floor = floor || std::strcmp(argv[i], "floor") == 0;
    stream = stream || std::strcmp(argv[i], "stream") == 0;
    chain = chain || std::strcmp(argv[i], "chain") == 0;
    ramp = ramp || std::strcmp(argv[i], "ramp") == 0;
    latency = latency || std::strcmp(argv[i], "latency") == 0;
    code = code || std::strcmp(argv[i], "code") == 0;
  }
  CK(hipSetDevice(0));
  hipDeviceProp_t prop;
  CK(hipGetDeviceProperties(&prop, 0));
  std::printf("device: %s, %d compute units\n", prop.name, prop.multiProcessorCount);
  hipStream_t st;
  CK(hipStreamCreate(&st));
  // one GEMV's weight bytes at 13824 x 5120 (codes + scales), 16 copies: beyond the 256 MB
  // memory-side cache
  const size_t copy_bytes = 13824ull * 2560 + 13824ull * 160;
  const int copies = 17;
  uint8_t *weights = nullptr;
  CK(hipMalloc(&weights, copy_bytes * copies));
  CK(hipMemset(weights, 0x5A, copy_bytes * copies));
  uint32_t *out = nullptr;
  CK(hipMalloc(&out, 1 << 20));
  CK(hipDeviceSynchronize());
  if (floor) {
    run_floor(st);
  }
  if (stream) {
    run_stream(st, weights, copy_bytes, copies, out);
  }
  if (chain) {
    run_chain(st, weights, copy_bytes, copies);
  }
  if (ramp) {
    run_ramp(st, weights, copy_bytes, copies);
  }
  if (latency) {
    run_latency(st);
  }
  if (code) {
    run_code(st);
  }
  CK(hipFree(weights));
  CK(hipFree(out));
  CK(hipStreamDestroy(st));
  std::printf("done\n");
  return 0;
}
