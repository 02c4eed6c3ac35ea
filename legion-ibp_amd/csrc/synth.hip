// Synthetic inputs generated on the GPU: power-law graphs, train sets, N(0,1)
// feature rows.  Stand-in for the reference's dataset tooling (dataset/,
// dataset_info.py), which needs network access.  Integer arithmetic on
// Philox4x32-10 words only, so a host implementation reproduces the graph bit
// for bit; the feature generator uses device transcendentals and is data, not
// part of any parity claim.
#include <algorithm>
#include <numeric>

#include "scan.hpp"

namespace lmi {

// degree(v) = first j with u <= cdf[j],  u = Philox(seed; v_lo, v_hi, 0x5eed0001, 0).x
static __global__ __launch_bounds__(256) void synth_degree_kernel(uint64_t seed, const uint32_t *cdf, int cdf_len,
                                                                  int64_t n, int32_t *deg) {
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < n; v += (int64_t)gridDim.x * blockDim.x) {
    const uint32_t u =
        philox4x32_10((uint32_t)v, (uint32_t)((uint64_t)v >> 32), 0x5eed0001u, 0u, (uint32_t)seed, (uint32_t)(seed >> 32)).x;
    int lo = 0, hi = cdf_len;  // first index with cdf[idx] >= u
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (cdf[mid] < u) lo = mid + 1; else hi = mid;
    }
    deg[v] = lo < cdf_len ? lo : cdf_len - 1;
  }
}

// 64-bit exclusive scan of int32 degrees by chunks: chunk totals on the host
// (n / 2^20 values), per-chunk device scans on 32-bit offsets.
static __global__ __launch_bounds__(256) void chunk_sum_kernel(const int32_t *deg, int64_t n, int64_t chunk,
                                                               unsigned long long *sums) {
  const int64_t c = blockIdx.x;
  const int64_t b = c * chunk, e = ((b + chunk < n) ? b + chunk : n);
  unsigned long long t = 0;
  for (int64_t i = b + threadIdx.x; i < e; i += blockDim.x) t += (unsigned long long)deg[i];
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) t += __shfl_down(t, d, kWave);
  __shared__ unsigned long long part[4];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = t;
  __syncthreads();
  if (threadIdx.x == 0) sums[c] = part[0] + part[1] + part[2] + part[3];
}

static __global__ __launch_bounds__(256) void chunk_scan_kernel(const int32_t *deg, int64_t n, int64_t chunk,
                                                                const unsigned long long *offs, int64_t *indptr) {
  // one block per chunk, sequential over 256-wide strips
  __shared__ int lds[256 / kWave + 1];
  const int64_t c = blockIdx.x;
  const int64_t b = c * chunk, e = ((b + chunk < n) ? b + chunk : n);
  long long carry = (long long)offs[c];
  for (int64_t s0 = b; s0 < e; s0 += 256 * 8) {
    const int64_t base = s0 + (int64_t)threadIdx.x * 8;
    int v[8], sum = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      v[j] = (base + j < e) ? deg[base + j] : 0;
      sum += v[j];
    }
    int total;
    long long run = carry + block_exclusive_scan<256>(sum, lds, total);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (base + j < e) indptr[base + j] = run;
      run += v[j];
    }
    carry += total;
  }
}

// neighbour of edge slot e: uniform node (mode 0) or the owner of a uniform edge
// slot (mode 1, degree-proportional), from 64 Philox bits.
static __global__ __launch_bounds__(256) void synth_indices_kernel(uint64_t seed, const int64_t *indptr, int64_t n_nodes,
                                                                   int64_t n_edges, int mode, int32_t *indices) {
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n_edges; e += (int64_t)gridDim.x * blockDim.x) {
    const Philox4 r =
        philox4x32_10((uint32_t)e, (uint32_t)((uint64_t)e >> 32), 0x5eed0002u, 0u, (uint32_t)seed, (uint32_t)(seed >> 32));
    const uint64_t x = (uint64_t)r.x | ((uint64_t)r.y << 32);
    if (mode == 0) {
      indices[e] = (int32_t)__umul64hi(x, (uint64_t)n_nodes);
    } else {
      const int64_t slot = (int64_t)__umul64hi(x, (uint64_t)n_edges);
      int64_t lo = 0, hi = n_nodes + 1;  // first index with indptr[idx] > slot
      while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (indptr[mid] <= slot) lo = mid + 1; else hi = mid;
      }
      indices[e] = (int32_t)(lo - 1);
    }
  }
}

// Box-Muller on two Philox words per pair of outputs.
static __global__ __launch_bounds__(256) void synth_features_kernel(uint64_t seed, void *rows, int64_t n_elems, int dtype) {
  const int64_t n_quads = (n_elems + 3) / 4;
  for (int64_t qd = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; qd < n_quads; qd += (int64_t)gridDim.x * blockDim.x) {
    const Philox4 r =
        philox4x32_10((uint32_t)qd, (uint32_t)((uint64_t)qd >> 32), 0x5eed0004u, 0u, (uint32_t)seed, (uint32_t)(seed >> 32));
    const float u0 = ((float)(r.x >> 8) + 0.5f) * (1.0f / 16777216.0f), u1 = ((float)(r.y >> 8) + 0.5f) * (1.0f / 16777216.0f);
    const float u2 = ((float)(r.z >> 8) + 0.5f) * (1.0f / 16777216.0f), u3 = ((float)(r.w >> 8) + 0.5f) * (1.0f / 16777216.0f);
    const float ra = sqrtf(-2.0f * logf(u0)), rb = sqrtf(-2.0f * logf(u2));
    float o[4] = {ra * cosf(6.2831853f * u1), ra * sinf(6.2831853f * u1), rb * cosf(6.2831853f * u3),
                  rb * sinf(6.2831853f * u3)};
    for (int k = 0; k < 4; ++k) {
      const int64_t i = qd * 4 + k;
      if (i >= n_elems) break;
      if (dtype == LMI_F16) reinterpret_cast<__half *>(rows)[i] = __float2half_rn(o[k]);
      else reinterpret_cast<float *>(rows)[i] = o[k];
    }
  }
}

}  // namespace lmi

using namespace lmi;

extern "C" int lmi_synth_graph(uint64_t seed, const uint32_t *cdf, int32_t cdf_len, int64_t n_nodes, int32_t mode,
                               int64_t **d_indptr, int32_t **d_indices, int64_t *n_edges) {
  if (!cdf || cdf_len < 1 || n_nodes < 1 || !d_indptr || !d_indices || !n_edges) LMI_FAIL(LMI_ERR_ARG, "bad synth_graph args");
  uint32_t *d_cdf = nullptr;
  int32_t *d_deg = nullptr;
  LMI_HIP(hipMalloc(&d_cdf, (size_t)cdf_len * 4));
  LMI_HIP(hipMemcpy(d_cdf, cdf, (size_t)cdf_len * 4, hipMemcpyHostToDevice));
  LMI_HIP(hipMalloc(&d_deg, (size_t)n_nodes * 4));
  hipLaunchKernelGGL(synth_degree_kernel, dim3(2048), dim3(256), 0, 0, seed, d_cdf, cdf_len, n_nodes, d_deg);
  LMI_HIP(hipGetLastError());
  const int64_t chunk = int64_t(1) << 20;
  const int64_t n_chunks = ceil_div(n_nodes, chunk);
  unsigned long long *d_sums = nullptr;
  LMI_HIP(hipMalloc(&d_sums, (size_t)n_chunks * 8));
  hipLaunchKernelGGL(chunk_sum_kernel, dim3((int)n_chunks), dim3(256), 0, 0, d_deg, n_nodes, chunk, d_sums);
  std::vector<unsigned long long> sums((size_t)n_chunks);
  LMI_HIP(hipMemcpy(sums.data(), d_sums, (size_t)n_chunks * 8, hipMemcpyDeviceToHost));
  unsigned long long total = 0;
  for (auto &x : sums) { const unsigned long long t = x; x = total; total += t; }
  LMI_HIP(hipMemcpy(d_sums, sums.data(), (size_t)n_chunks * 8, hipMemcpyHostToDevice));
  int64_t *indptr = nullptr;
  LMI_HIP(hipMalloc(&indptr, (size_t)(n_nodes + 1) * 8));
  hipLaunchKernelGGL(chunk_scan_kernel, dim3((int)n_chunks), dim3(256), 0, 0, d_deg, n_nodes, chunk, d_sums, indptr);
  const long long tot = (long long)total;
  LMI_HIP(hipMemcpy(indptr + n_nodes, &tot, 8, hipMemcpyHostToDevice));
  int32_t *indices = nullptr;
  LMI_HIP(hipMalloc(&indices, (size_t)std::max<long long>(tot, 1) * 4));
  if (tot > 0)
    hipLaunchKernelGGL(synth_indices_kernel, dim3(8192), dim3(256), 0, 0, seed, indptr, n_nodes, (int64_t)tot, mode, indices);
  LMI_HIP(hipGetLastError());
  LMI_HIP(hipDeviceSynchronize());
  (void)hipFree(d_cdf); (void)hipFree(d_deg); (void)hipFree(d_sums);
  *d_indptr = indptr;
  *d_indices = indices;
  *n_edges = tot;
  return LMI_OK;
}

// n_train distinct ids: stratum p = (i * P) mod n_train covers
// [p * stride, (p + 1) * stride), the id is a Philox-uniform point inside it.
extern "C" int lmi_synth_trainset(uint64_t seed, int64_t n_nodes, int32_t n_train, int32_t *host_ids) {
  if (n_train < 1 || n_nodes < n_train || !host_ids) LMI_FAIL(LMI_ERR_ARG, "bad synth_trainset args");
  const uint32_t stride = (uint32_t)(n_nodes / n_train);
  uint64_t P = 1000003;
  while (std::gcd<uint64_t, uint64_t>(P, (uint64_t)n_train) != 1) ++P;
  for (int32_t i = 0; i < n_train; ++i) {
    const uint32_t p = (uint32_t)(((uint64_t)i * P) % (uint64_t)n_train);
    // host-side Philox4x32-10, same rounds as the device function
    uint32_t c0 = p, c1 = 0, c2 = 0x5eed0003u, c3 = 0, k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
    for (int r = 0; r < 10; ++r) {
      const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
      const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
      c1 = (uint32_t)p1; c3 = (uint32_t)p0; c0 = n0; c2 = n2;
      k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    host_ids[i] = (int32_t)(p * stride + (uint32_t)(((uint64_t)c0 * stride) >> 32));
  }
  return LMI_OK;
}

extern "C" int lmi_synth_features(uint64_t seed, void *rows, int64_t n_rows, int32_t dim, int32_t dtype) {
  if (!rows || n_rows < 1 || dim < 1) LMI_FAIL(LMI_ERR_ARG, "bad synth_features args");
  void *dptr = rows;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, rows) == hipSuccess && attr.type == hipMemoryTypeHost) {
    LMI_HIP(hipHostGetDevicePointer(&dptr, rows, 0));
  } else {
    (void)hipGetLastError();
  }
  hipLaunchKernelGGL(synth_features_kernel, dim3(8192), dim3(256), 0, 0, seed, dptr, n_rows * (int64_t)dim, dtype);
  LMI_HIP(hipGetLastError());
  LMI_HIP(hipDeviceSynchronize());
  return LMI_OK;
}
