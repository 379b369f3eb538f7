// Host-only pieces of the C ABI: error reporting, pinned mapped allocations and
// the CPU row gather.
//
// Reference for the CPU gather: cache_hub/gather/gather_cpu.cpp:21-170
// (gather_kv_out_cpu: at::parallel_for over (batch, head), prefetch + memcpy).
#include "pkv_common.h"

#include <stdarg.h>

#include <string>
#include <thread>
#include <vector>

static thread_local std::string g_last_error;

void pkv_set_error(const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
}

extern "C" int pkv_version(void) { return 1; }

extern "C" size_t pkv_struct_bytes(int which) {
  switch (which) {
    case 0: return sizeof(pkv_attn_segment);
    case 1: return sizeof(pkv_attn_args);
    case 2: return sizeof(pkv_retrieve_args);
    case 3: return sizeof(pkv_adaptive_args);
    default: return 0;
  }
}

extern "C" const char *pkv_last_error(void) { return g_last_error.c_str(); }

extern "C" int pkv_host_alloc_mapped(size_t bytes, void **host_ptr) {
  PKV_REQUIRE(host_ptr != nullptr && bytes > 0, "pkv_host_alloc_mapped: bad arguments");
  void *p = nullptr;
  hipError_t e = hipHostMalloc(&p, bytes, hipHostMallocMapped | hipHostMallocPortable);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    pkv_set_error("hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    return PKV_ENOMEM;
  }
  *host_ptr = p;
  return PKV_OK;
}

extern "C" int pkv_host_free(void *host_ptr) {
  if (!host_ptr) return PKV_OK;
  PKV_HIP(hipHostFree(host_ptr));
  return PKV_OK;
}

extern "C" int pkv_host_device_pointer(const void *host_ptr, void **dev_ptr) {
  PKV_REQUIRE(host_ptr && dev_ptr, "pkv_host_device_pointer: null pointer");
  void *d = nullptr;
  hipError_t e = hipHostGetDevicePointer(&d, const_cast<void *>(host_ptr), 0);
  if (e != hipSuccess || !d) {
    (void)hipGetLastError();
    pkv_set_error("not pinned, device-mapped host memory (%s)", hipGetErrorString(e));
    return PKV_EINVAL;
  }
  *dev_ptr = d;
  return PKV_OK;
}

extern "C" int pkv_gather_cpu(const void *src, const int64_t *ss, const int64_t *index, void *out, const int64_t *os,
                              int64_t B, int64_t H, int64_t N, int64_t D, int64_t K, int elem_bytes, int n_threads) {
  PKV_REQUIRE(src && ss && index && out && os, "pkv_gather_cpu: null pointer");
  PKV_REQUIRE(B > 0 && H > 0 && N > 0 && D > 0 && K >= 0 && elem_bytes > 0, "pkv_gather_cpu: bad shape");
  const int64_t total = B * H * K;
  for (int64_t i = 0; i < total; ++i) {
    if (index[i] < 0 || index[i] >= N) {
      pkv_set_error("index %lld is out of bounds for dimension 2 with size %lld", (long long)index[i], (long long)N);
      return PKV_EINVAL;
    }
  }
  const bool contiguous = ss[3] == 1 && os[3] == 1;
  const size_t row_bytes = (size_t)D * (size_t)elem_bytes;
  auto work = [&](int64_t bh0, int64_t bh1) {
    for (int64_t bh = bh0; bh < bh1; ++bh) {
      const int64_t b = bh / H, h = bh - b * H;
      const char *sb = (const char *)src + (b * ss[0] + h * ss[1]) * elem_bytes;
      char *ob = (char *)out + (b * os[0] + h * os[1]) * elem_bytes;
      const int64_t *ib = index + bh * K;
      for (int64_t k = 0; k < K; ++k) {
        if (k + 4 < K) __builtin_prefetch(sb + ib[k + 4] * ss[2] * elem_bytes, 0, 0);
        const char *srow = sb + ib[k] * ss[2] * elem_bytes;
        char *orow = ob + k * os[2] * elem_bytes;
        if (contiguous) {
          memcpy(orow, srow, row_bytes);
        } else {
          for (int64_t d = 0; d < D; ++d) memcpy(orow + d * os[3] * elem_bytes, srow + d * ss[3] * elem_bytes, (size_t)elem_bytes);
        }
      }
    }
  };
  const int64_t bh_total = B * H;
  int nt = n_threads < 1 ? 1 : n_threads;
  if (nt > bh_total) nt = (int)bh_total;
  if (nt <= 1) {
    work(0, bh_total);
  } else {
    std::vector<std::thread> th;
    const int64_t per = (bh_total + nt - 1) / nt;
    for (int t = 0; t < nt; ++t) {
      const int64_t a = t * per, e = (a + per < bh_total) ? a + per : bh_total;
      if (a < e) th.emplace_back(work, a, e);
    }
    for (auto &t : th) t.join();
  }
  return PKV_OK;
}
