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

// TO_CACHE: layers -> cache; otherwise cache -> layers.
template <typename V, bool TO_CACHE>
__global__ __launch_bounds__(256) void reorg_kernel(const ReorgArgs a) {
  const int64_t tok = blockIdx.x;
  const int vec_per_row = (int)(a.row_bytes / sizeof(V));
  const int total = vec_per_row * a.n_layers;
  char* cbase = reinterpret_cast<char*>(a.cache) + tok * a.cache_token_bytes + a.slot0_bytes;
  auto at = [&](int i, V*& lp, V*& cp) {
    const int l = i / vec_per_row, w = i - l * vec_per_row;
    lp = reinterpret_cast<V*>(reinterpret_cast<char*>(a.layer[l]) + tok * a.row_bytes) + w;
    cp = reinterpret_cast<V*>(cbase + (int64_t)l * a.row_bytes) + w;
  };
  // Streamed once in, once out: nothing here is read again by this launch.  Four loads go out before the first
  // store so that a thread keeps 64 bytes in flight.
  constexpr int U = 4;
  int i = threadIdx.x;
  for (; i + (U - 1) * 256 < total; i += U * 256) {
    V *lp[U], *cp[U], x[U];
#pragma unroll
    for (int u = 0; u < U; u++) at(i + u * 256, lp[u], cp[u]);
#pragma unroll
    for (int u = 0; u < U; u++) x[u] = __builtin_nontemporal_load(TO_CACHE ? lp[u] : cp[u]);
#pragma unroll
    for (int u = 0; u < U; u++) __builtin_nontemporal_store(x[u], TO_CACHE ? cp[u] : lp[u]);
  }
  for (; i < total; i += 256) {
    V *lp, *cp;
    at(i, lp, cp);
    __builtin_nontemporal_store(__builtin_nontemporal_load(TO_CACHE ? lp : cp), TO_CACHE ? cp : lp);
  }
}

typedef int v4i __attribute__((ext_vector_type(4)));

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
    const dim3 grid((unsigned)n_tokens), block(256);
    if (wide) {
      if (to_cache)
        hipLaunchKernelGGL((reorg_kernel<v4i, true>), grid, block, 0, stream, a);
      else
        hipLaunchKernelGGL((reorg_kernel<v4i, false>), grid, block, 0, stream, a);
    } else {
      if (to_cache)
        hipLaunchKernelGGL((reorg_kernel<uint16_t, true>), grid, block, 0, stream, a);
      else
        hipLaunchKernelGGL((reorg_kernel<uint16_t, false>), grid, block, 0, stream, a);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace moda
