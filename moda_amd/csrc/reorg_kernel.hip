// Depth-KV reorganisation: per-layer [B,T,H,D] tensors <-> token-major depth
// cache [B, T*L, H, D] (row t*L + l = layer l of token t), the layout the
// attention kernels read; the permutation of vision_tasks/deit/models.py:361-375
// and its transpose.  Pure HBM copy: one workgroup per token moves the
// n_layers * H * D contiguous cache bytes of that token with 16-byte accesses,
// so cache traffic is fully coalesced and each layer row is one contiguous run.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace moda {

constexpr int kMaxLayersPerLaunch = 64;

struct ReorgArgs {
  void* layer[kMaxLayersPerLaunch];
  void* cache;
  int64_t n_tokens;     // B * T
  int64_t row_bytes;    // H * D * sizeof(elem)
  int64_t cache_token_bytes;  // L_total * row_bytes
  int64_t slot0_bytes;  // slot0 * row_bytes
  int n_layers;
};

typedef int v4i __attribute__((ext_vector_type(4)));

// TO_CACHE: layers -> cache; otherwise cache -> layers.  One workgroup per token.  A thread issues U loads before
// its first store (the launcher picks the workgroup size and U so that most shapes take one such batch).  STREAM:
// nontemporal accesses on both sides.
template <typename V, bool TO_CACHE, int U, int NT, bool STREAM>
__global__ __launch_bounds__(NT) void reorg_kernel(const ReorgArgs a) {
  const int64_t tok = blockIdx.x;
  const int vec_per_row = (int)(a.row_bytes / sizeof(V));
  const int total = vec_per_row * a.n_layers;
  char* cbase = reinterpret_cast<char*>(a.cache) + tok * a.cache_token_bytes + a.slot0_bytes;
  auto ends = [&](int i, V*& src, V*& dst) {
    const int l = i / vec_per_row, w = i - l * vec_per_row;
    V* lp = reinterpret_cast<V*>(reinterpret_cast<char*>(a.layer[l]) + tok * a.row_bytes) + w;
    V* cp = reinterpret_cast<V*>(cbase + (int64_t)l * a.row_bytes) + w;
    src = TO_CACHE ? lp : cp;
    dst = TO_CACHE ? cp : lp;
  };
  auto get = [](const V* p) { return STREAM ? __builtin_nontemporal_load(p) : *p; };
  auto put = [](V x, V* p) {
    if (STREAM)
      __builtin_nontemporal_store(x, p);
    else
      *p = x;
  };
  int i = threadIdx.x;
  for (; i + (U - 1) * NT < total; i += U * NT) {
    V *src[U], *dst[U], x[U];
#pragma unroll
    for (int u = 0; u < U; u++) ends(i + u * NT, src[u], dst[u]);
#pragma unroll
    for (int u = 0; u < U; u++) x[u] = get(src[u]);
#pragma unroll
    for (int u = 0; u < U; u++) put(x[u], dst[u]);
  }
  for (; i < total; i += NT) {
    V *src, *dst;
    ends(i, src, dst);
    put(get(src), dst);
  }
}

template <typename V, bool TO_CACHE, int NT, bool STREAM>
void launch_reorg_batch(const ReorgArgs& a, int64_t n_tokens, int per, hipStream_t stream) {
  const dim3 grid((unsigned)n_tokens), block(NT);
  if (per <= 1)
    hipLaunchKernelGGL((reorg_kernel<V, TO_CACHE, 1, NT, STREAM>), grid, block, 0, stream, a);
  else if (per == 2)
    hipLaunchKernelGGL((reorg_kernel<V, TO_CACHE, 2, NT, STREAM>), grid, block, 0, stream, a);
  else if (per == 3)
    hipLaunchKernelGGL((reorg_kernel<V, TO_CACHE, 3, NT, STREAM>), grid, block, 0, stream, a);
  else
    hipLaunchKernelGGL((reorg_kernel<V, TO_CACHE, 4, NT, STREAM>), grid, block, 0, stream, a);
}

// What one launch moves (read + written) against the 256 MB of memory-side cache: a copy that fits stays there for
// the attention kernels that read the cache next; a larger one would only push itself out, and streams past.
constexpr int64_t kStreamAboveBytes = 256ll << 20;

template <typename V, bool TO_CACHE, bool STREAM>
void launch_reorg_sized(const ReorgArgs& a, int64_t n_tokens, hipStream_t stream) {
  const int64_t total = a.row_bytes / (int64_t)sizeof(V) * a.n_layers;
  // 512 threads when that still leaves every thread two accesses, else 256; then as many loads per batch (up to
  // four) as cover the token in one trip
  if (total >= 1024)
    launch_reorg_batch<V, TO_CACHE, 512, STREAM>(a, n_tokens, (int)((total + 511) / 512), stream);
  else
    launch_reorg_batch<V, TO_CACHE, 256, STREAM>(a, n_tokens, (int)((total + 255) / 256), stream);
}

template <typename V, bool TO_CACHE>
void launch_reorg_kernel(const ReorgArgs& a, int64_t n_tokens, hipStream_t stream) {
  if (2 * n_tokens * a.n_layers * a.row_bytes > kStreamAboveBytes)
    launch_reorg_sized<V, TO_CACHE, true>(a, n_tokens, stream);
  else
    launch_reorg_sized<V, TO_CACHE, false>(a, n_tokens, stream);
}

hipError_t launch_reorg(void* const* layers, int64_t n_layers, int64_t slot0, int64_t L_total, int64_t n_tokens,
                        int64_t row_bytes, void* cache, bool to_cache, hipStream_t stream) {
  if (n_tokens == 0 || n_layers == 0 || row_bytes == 0) return hipSuccess;
  for (int64_t l0 = 0; l0 < n_layers; l0 += kMaxLayersPerLaunch) {
    ReorgArgs a;
    a.n_layers = (int)((n_layers - l0) < kMaxLayersPerLaunch ? (n_layers - l0) : kMaxLayersPerLaunch);
    for (int i = 0; i < a.n_layers; i++) a.layer[i] = layers[l0 + i];
    for (int i = a.n_layers; i < kMaxLayersPerLaunch; i++) a.layer[i] = nullptr;
    a.cache = cache;
    a.n_tokens = n_tokens;
    a.row_bytes = row_bytes;
    a.cache_token_bytes = L_total * row_bytes;
    a.slot0_bytes = (slot0 + l0) * row_bytes;
    bool wide = (row_bytes % 16 == 0) && ((uintptr_t)cache % 16 == 0);
    for (int i = 0; i < a.n_layers; i++) wide = wide && ((uintptr_t)a.layer[i] % 16 == 0);
    if (wide) {
      if (to_cache)
        launch_reorg_kernel<v4i, true>(a, n_tokens, stream);
      else
        launch_reorg_kernel<v4i, false>(a, n_tokens, stream);
    } else {
      if (to_cache)
        launch_reorg_kernel<uint16_t, true>(a, n_tokens, stream);
      else
        launch_reorg_kernel<uint16_t, false>(a, n_tokens, stream);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace moda
