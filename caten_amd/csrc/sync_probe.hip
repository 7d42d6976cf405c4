// Measures what bounds a decode step that is a chain of DEPENDENT phases on gfx950: the cost of a kernel
// boundary inside a hipGraph, and the cost of the alternatives to one (grid barriers and flags inside a
// persistent kernel).  Prints one line per measurement.  Every wait in every kernel is bounded: a waiter that
// runs out of spins raises a flag the host reports, and all kernels exit normally either way.
//
//   chain     N dependent kernel nodes in one hipGraph: empty; reading what the predecessor wrote and writing
//             for the successor (one memory round trip); the same over 256 workgroups
//   barrier   256 workgroups of a persistent kernel meeting R times:
//               one     every workgroup adds to ONE device-scope counter and polls it
//               tree    arrivals per XCD on counters in that XCD's L2 (atomics without device-scope bits),
//                       one device-scope arrival per XCD, the release fanned out the same way
//   signal    one workgroup hands a value to another and gets it back (half a round trip = one hop):
//               same XCD through its L2; different XCDs through device-scope atomics
//   relay     ONE launch of P x W workgroups, far more than fit the chip at once: the W workgroups of phase p
//             wait (device-scope counter) until all of phase p-1 have published, read the whole vector phase
//             p-1 wrote (release / acquire fences), write their slice of the next one and publish.  Workgroups
//             are dispatched in index order, so whatever a resident workgroup waits for is resident or done.
//             Time per phase = what a dependent phase costs WITHOUT a kernel boundary.
//
// Build: make -C caten_amd/csrc sync_probe     Run: caten_amd/sync_probe.bin [rounds]
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

#include <vector>

#define CHECK(e)                                                                                  \
  do {                                                                                            \
    hipError_t _e = (e);                                                                          \
    if (_e != hipSuccess) {                                                                       \
      fprintf(stderr, "%s:%d: %s -> %s\n", __FILE__, __LINE__, #e, hipGetErrorString(_e));        \
      exit(1);                                                                                    \
    }                                                                                             \
  } while (0)

constexpr int kSpinLimit = 1 << 20;  // polls before a waiter gives up (a poll is ~1 us at worst)
constexpr int kXcds = 8;
constexpr int kLine = 64;  // ints per 256-byte slot: every counter and flag sits alone in its cache lines

__device__ __forceinline__ int xcd_id() { return (int)__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20); }

// ---- atomics at the two scopes ----
// device scope: visible to every XCD (performed behind the L2s)
__device__ __forceinline__ int dev_add(int *p, int v) { return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ int dev_load(int *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void dev_store(int *p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// L2 of the issuing XCD: a read-modify-write without device-scope bits (a plain load could be served by the
// compute unit's own L1)
__device__ __forceinline__ int l2_add(int *p, int v) { return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }
__device__ __forceinline__ int l2_load(int *p) { return l2_add(p, 0); }

// Polls until ready() holds.  Gives up after kSpinLimit polls (raising *fail for the host and for every other
// waiter, which look at it now and then); returns false then and the caller stops waiting for good.
template <class F>
__device__ __forceinline__ bool wait_until(F ready, int *fail) {
  int spins = 0;
  while (!ready()) {
    if (++spins > kSpinLimit) {
      dev_store(fail, 1);
      return false;
    }
    if ((spins & 255) == 0 && dev_load(fail)) return false;
  }
  return true;
}

// ------------------------------------------------------------------ chain
__global__ void k_empty() {}
__global__ void k_hop(const float *in, float *out) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  out[i] = in[i] + 1.0f;
}

static float time_graph(hipStream_t st, hipGraphExec_t g, int reps) {
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  for (int i = 0; i < 3; i++) CHECK(hipGraphLaunch(g, st));
  CHECK(hipStreamSynchronize(st));
  CHECK(hipEventRecord(a, st));
  for (int i = 0; i < reps; i++) CHECK(hipGraphLaunch(g, st));
  CHECK(hipEventRecord(b, st));
  CHECK(hipEventSynchronize(b));
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, a, b));
  CHECK(hipEventDestroy(a));
  CHECK(hipEventDestroy(b));
  return ms * 1e3f / reps;
}

static void chain(hipStream_t st, int nodes, int grid, int block, bool hop, const char *what) {
  float *buf[2];
  CHECK(hipMalloc(&buf[0], sizeof(float) * 256 * 1024));
  CHECK(hipMalloc(&buf[1], sizeof(float) * 256 * 1024));
  CHECK(hipMemset(buf[0], 0, sizeof(float) * 256 * 1024));
  hipGraph_t g;
  hipGraphExec_t ex;
  CHECK(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
  for (int i = 0; i < nodes; i++) {
    if (hop) hipLaunchKernelGGL(k_hop, dim3(grid), dim3(block), 0, st, buf[i & 1], buf[(i + 1) & 1]);
    else hipLaunchKernelGGL(k_empty, dim3(grid), dim3(block), 0, st);
  }
  CHECK(hipStreamEndCapture(st, &g));
  CHECK(hipGraphInstantiate(&ex, g, nullptr, nullptr, 0));
  const float us = time_graph(st, ex, 50);
  printf("chain    %-58s %4d nodes  %8.2f us/graph  %6.3f us/node\n", what, nodes, us, us / nodes);
  CHECK(hipGraphExecDestroy(ex));
  CHECK(hipGraphDestroy(g));
  CHECK(hipFree(buf[0]));
  CHECK(hipFree(buf[1]));
}

// ------------------------------------------------------------------ barrier
// state: [0] device-scope counter, [1] device-scope release generation, [2] give-up flag,
//        [4 + k] arrivals of XCD k (its L2), [12 + k] release generation of XCD k (its L2), [20 + k] members of XCD k
__global__ __launch_bounds__(256) void k_barrier_one(int *s, int rounds) {
  int *count = s, *fail = s + 2 * kLine;
  const int n = gridDim.x;
  bool alive = true;
  for (int r = 1; r <= rounds; r++) {
    __syncthreads();
    if (threadIdx.x == 0 && alive) {
      dev_add(count, 1);
      alive = wait_until([&] { return dev_load(count) >= r * n; }, fail);
    }
  }
}

// members of each XCD are counted by a first kernel (k_census); this one trusts the counts
__global__ __launch_bounds__(256) void k_barrier_tree(int *s, int rounds) {
  int *root = s, *gen = s + kLine, *fail = s + 2 * kLine;
  const int k = xcd_id() & (kXcds - 1);
  int *arrive = s + (4 + k) * kLine, *lgen = s + (12 + k) * kLine;
  const int members = s[(20 + k) * kLine];
  int live = 0;
  for (int q = 0; q < kXcds; q++) live += s[(20 + q) * kLine] > 0;
  bool alive = true;
  for (int r = 1; r <= rounds; r++) {
    __syncthreads();
    if (threadIdx.x == 0 && alive) {
      const int t = l2_add(arrive, 1);
      if (t == r * members - 1) {
        // last of this XCD: one device-scope arrival, then wait for the device-wide release and pass it on
        const int g = dev_add(root, 1);
        if (g == r * live - 1) dev_store(gen, r);
        else alive = wait_until([&] { return dev_load(gen) >= r; }, fail);
        l2_add(lgen, 1);
      } else {
        alive = wait_until([&] { return l2_load(lgen) >= r; }, fail);
      }
    }
  }
}

__global__ void k_census(int *s) {
  if (threadIdx.x == 0) l2_add(s + (20 + (xcd_id() & (kXcds - 1))) * kLine, 1);
}

// ------------------------------------------------------------------ signal
// Two workgroups, A and B, picked by a census of (XCD, arrival order): A bumps `ping`, B answers on `pong`.
// s: [0] ping, [1] pong, [2] give-up, [3] roles taken, [4 + k] arrival order on XCD k
template <bool SAME_XCD>
__global__ void k_signal(int *s, int rounds, int *role_out) {
  if (threadIdx.x != 0) return;
  int *ping = s, *pong = s + kLine, *fail = s + 2 * kLine;
  const int k = xcd_id() & (kXcds - 1);
  const int order = l2_add(s + (4 + k) * kLine, 1);
  // A = first arrival on the XCD of block 0 ... simplest: block 0 is A; B = the first block that finds itself
  // on the wanted side and wins the device-scope claim
  int role = -1;
  if (blockIdx.x == 0) {
    role = 0;
    dev_store(s + 3 * kLine + 1, k + 1);  // A's XCD, +1
  } else {
    int spins = 0, ax = 0;
    while ((ax = dev_load(s + 3 * kLine + 1)) == 0 && ++spins < 4096) {}
    const bool wanted = SAME_XCD ? (ax - 1 == k) : (ax - 1 != k);
    if (ax && wanted && dev_add(s + 3 * kLine, 1) == 0) role = 1;
  }
  (void)order;
  if (role < 0) return;
  role_out[role] = k;
  for (int r = 1; r <= rounds; r++) {
    bool ok;
    if (role == 0) {
      if (SAME_XCD) {
        l2_add(ping, 1);
        ok = wait_until([&] { return l2_load(pong) >= r; }, fail);
      } else {
        dev_add(ping, 1);
        ok = wait_until([&] { return dev_load(pong) >= r; }, fail);
      }
    } else {
      if (SAME_XCD) {
        ok = wait_until([&] { return l2_load(ping) >= r; }, fail);
        l2_add(pong, 1);
      } else {
        ok = wait_until([&] { return dev_load(ping) >= r; }, fail);
        dev_add(pong, 1);
      }
    }
    if (!ok) return;
  }
}

// ------------------------------------------------------------------ relay
// s: [0] give-up flag, [1 + p] arrivals of phase p (one 256-byte slot each); vec: two buffers of n floats
// FINE = false: plain loads / stores ordered by device-scope release / acquire FENCES (which write back and
// invalidate the whole L2).  FINE = true: the vector itself moves through device-scope accesses (stores written
// through, loads served behind the L2), so publishing only waits for the workgroup's own stores.
__device__ __forceinline__ float2 dev_load2(const float *p) {
  const unsigned long long u = __hip_atomic_load((const unsigned long long *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_float2(__uint_as_float((unsigned)u), __uint_as_float((unsigned)(u >> 32)));
}
__device__ __forceinline__ void dev_store1(float *p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

template <int NT, bool FINE>
__global__ __launch_bounds__(NT) void k_relay(int *s, float *vec, int n, int W, float *check) {
  __shared__ float red[16];
  __shared__ int go;
  int *fail = s;
  const int p = blockIdx.x / W, j = blockIdx.x % W;
  const int tid = threadIdx.x;
  if (p > 0) {
    if (tid == 0) {
      int *cnt = s + p * kLine;  // arrivals of phase p - 1
      go = wait_until([&] { return dev_load(cnt) >= W; }, fail) ? 1 : 0;
    }
    __syncthreads();
    if (!go) return;
    if (FINE) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    else __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  // read the whole previous vector
  const float *src = vec + (size_t)((p + 1) & 1) * n;
  float acc = 0.0f;
  if (p > 0) {
    if (FINE) {
      for (int i = tid; i < n / 2; i += NT) {
        const float2 v = dev_load2(src + 2 * i);
        acc += v.x + v.y;
      }
    } else {
      for (int i = tid; i < n / 4; i += NT) {
        const float4 v = ((const float4 *)src)[i];
        acc += (v.x + v.y) + (v.z + v.w);
      }
    }
  }
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if ((tid & 63) == 0) red[tid >> 6] = acc;
  __syncthreads();
  float tot = 0.0f;
  for (int w = 0; w < NT / 64; w++) tot += red[w];
  // write this workgroup's slice of the next vector: every element = mean of the previous vector + 1
  float *dst = vec + (size_t)(p & 1) * n;
  const int per = n / W;
  const float val = (p > 0 ? tot / (float)n : 0.0f) + 1.0f;
  for (int i = tid; i < per; i += NT) {
    if (FINE) dev_store1(dst + j * per + i, val);
    else dst[j * per + i] = val;
  }
  if (check && tid == 0 && j == 0) check[p] = val;
  if (FINE) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  else __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
  __syncthreads();
  if (tid == 0) dev_add(s + (p + 1) * kLine, 1);
}

static void relay(hipStream_t st, int P, int W, int nt, int n, bool fine) {
  int *s;
  float *vec, *check;
  const size_t sb = sizeof(int) * kLine * (size_t)(P + 2);
  CHECK(hipMalloc(&s, sb));
  CHECK(hipMalloc(&vec, sizeof(float) * 2 * n));
  CHECK(hipMalloc(&check, sizeof(float) * P));
  float best = 1e30f;
  std::vector<float> h(P);
  int gave_up = 0;
  bool ok = true;
  for (int rep = 0; rep < 5; rep++) {
    CHECK(hipMemset(s, 0, sb));
    CHECK(hipMemset(vec, 0, sizeof(float) * 2 * n));
    CHECK(hipStreamSynchronize(st));
    hipEvent_t a, b;
    CHECK(hipEventCreate(&a));
    CHECK(hipEventCreate(&b));
    CHECK(hipEventRecord(a, st));
    if (nt == 1024 && fine) hipLaunchKernelGGL((k_relay<1024, true>), dim3(P * W), dim3(1024), 0, st, s, vec, n, W, check);
    else if (nt == 1024) hipLaunchKernelGGL((k_relay<1024, false>), dim3(P * W), dim3(1024), 0, st, s, vec, n, W, check);
    else if (fine) hipLaunchKernelGGL((k_relay<256, true>), dim3(P * W), dim3(256), 0, st, s, vec, n, W, check);
    else hipLaunchKernelGGL((k_relay<256, false>), dim3(P * W), dim3(256), 0, st, s, vec, n, W, check);
    CHECK(hipEventRecord(b, st));
    CHECK(hipEventSynchronize(b));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, a, b));
    if (ms * 1e3f < best) best = ms * 1e3f;
    CHECK(hipMemcpy(&gave_up, s, sizeof(int), hipMemcpyDeviceToHost));
    CHECK(hipMemcpy(h.data(), check, sizeof(float) * P, hipMemcpyDeviceToHost));
    for (int p = 0; p < P; p++) ok = ok && h[p] == (float)(p + 1);  // every phase saw all of its predecessor
    CHECK(hipEventDestroy(a));
    CHECK(hipEventDestroy(b));
    if (gave_up) break;
  }
  char what[96];
  snprintf(what, sizeof(what), "%s %d phases x %d workgroups of %d", fine ? "device-scope accesses," : "fences,", P, W, nt);
  printf("relay    %-58s %5d workgroups %8.2f us total  %6.3f us/phase  values %s%s\n", what, P * W, best, best / P,
         ok ? "right" : "WRONG", gave_up ? "  (GAVE UP: a waiter ran out of spins)" : "");
  CHECK(hipFree(s));
  CHECK(hipFree(vec));
  CHECK(hipFree(check));
}

static float time_kernel(hipStream_t st, void (*launch)(hipStream_t, void *), void *ctx) {
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  CHECK(hipEventRecord(a, st));
  launch(st, ctx);
  CHECK(hipEventRecord(b, st));
  CHECK(hipEventSynchronize(b));
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, a, b));
  CHECK(hipEventDestroy(a));
  CHECK(hipEventDestroy(b));
  return ms * 1e3f;
}

struct Ctx {
  int *s;
  int rounds;
  int variant;
  int *roles;
};

static void run_barrier(hipStream_t st, void *p) {
  Ctx *c = (Ctx *)p;
  if (c->variant == 0) hipLaunchKernelGGL(k_barrier_one, dim3(256), dim3(256), 0, st, c->s, c->rounds);
  else hipLaunchKernelGGL(k_barrier_tree, dim3(256), dim3(256), 0, st, c->s, c->rounds);
}
static void run_signal(hipStream_t st, void *p) {
  Ctx *c = (Ctx *)p;
  if (c->variant == 0) hipLaunchKernelGGL(k_signal<true>, dim3(32), dim3(64), 0, st, c->s, c->rounds, c->roles);
  else hipLaunchKernelGGL(k_signal<false>, dim3(32), dim3(64), 0, st, c->s, c->rounds, c->roles);
}

int main(int argc, char **argv) {
  const int rounds = argc > 1 ? atoi(argv[1]) : 200;
  CHECK(hipSetDevice(0));
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  printf("device   %s, %d compute units\n", prop.name, prop.multiProcessorCount);
  hipStream_t st;
  CHECK(hipStreamCreate(&st));

  chain(st, 62, 1, 64, false, "empty kernel, 1 workgroup of 64");
  chain(st, 62, 256, 256, false, "empty kernel, 256 workgroups of 256");
  chain(st, 62, 1, 64, true, "reads what the predecessor wrote, writes; 1 workgroup of 64");
  chain(st, 62, 256, 256, true, "reads what the predecessor wrote, writes; 256 workgroups of 256");
  chain(st, 39, 256, 256, true, "the same, 39 nodes");

  const size_t state_bytes = sizeof(int) * kLine * 32;
  int *s, *roles;
  CHECK(hipMalloc(&s, state_bytes));
  CHECK(hipMalloc(&roles, 256));
  std::vector<int> h(kLine * 32);
  for (int variant = 0; variant < 2; variant++) {
    CHECK(hipMemset(s, 0, state_bytes));
    hipLaunchKernelGGL(k_census, dim3(256), dim3(256), 0, st, s);
    CHECK(hipStreamSynchronize(st));
    Ctx c = {s, rounds, variant, roles};
    const float us = time_kernel(st, run_barrier, &c);
    CHECK(hipMemcpy(h.data(), s, state_bytes, hipMemcpyDeviceToHost));
    printf("barrier  %-58s %4d rounds %8.2f us total  %6.3f us/barrier%s   workgroups per XCD:", variant == 0 ? "one device-scope counter, 256 workgroups" : "per-XCD L2 counters + device-scope root, 256 workgroups",
           rounds, us, us / rounds, h[2 * kLine] ? "  (GAVE UP: a waiter ran out of spins)" : "");
    for (int k = 0; k < kXcds; k++) printf(" %d", h[(20 + k) * kLine]);
    printf("\n");
  }
  for (int variant = 0; variant < 2; variant++) {
    CHECK(hipMemset(s, 0, state_bytes));
    CHECK(hipMemset(roles, 0xff, 256));
    Ctx c = {s, rounds, variant, roles};
    const float us = time_kernel(st, run_signal, &c);
    int r[2];
    CHECK(hipMemcpy(r, roles, sizeof(r), hipMemcpyDeviceToHost));
    CHECK(hipMemcpy(h.data(), s, state_bytes, hipMemcpyDeviceToHost));
    printf("signal   %-58s %4d rounds %8.2f us total  %6.3f us/hop (XCD %d <-> XCD %d)%s\n",
           variant == 0 ? "two workgroups of one XCD, through its L2" : "two workgroups of different XCDs, device-scope atomics", rounds, us,
           us / rounds / 2, r[0], r[1], (h[2 * kLine] || r[1] < 0) ? "  (GAVE UP or no partner)" : "");
  }
  CHECK(hipFree(s));
  CHECK(hipFree(roles));
  for (int fine = 0; fine < 2; fine++) {
    relay(st, 8, 48, 1024, 768, fine);    // all resident
    relay(st, 40, 48, 1024, 768, fine);   // 1920 workgroups of 1024: several times what the chip holds
    relay(st, 40, 12, 1024, 768, fine);
    relay(st, 40, 192, 256, 768, fine);
    relay(st, 200, 48, 1024, 768, fine);
    relay(st, 200, 48, 256, 768, fine);
  }
  CHECK(hipStreamDestroy(st));
  return 0;
}
