// Argument fuzzer for the host side of libarctic_mi355x's C ABI, meant to be built from the library's sources
// with AddressSanitizer and UBSan on the host pass (tests/test_abi_sanitizers.py does that) and run on a machine
// WITHOUT a GPU: every entry point is called with seeded random sizes, strides, type codes and pointers (fake
// device addresses that the host never reads, NULL, misaligned ones; per-layer host tables allocated with exactly
// the number of entries the call names).  A call may be turned away or may get as far as the launch, which
// fails for want of a device; either way it has to return a code, leave a message for every failure and trip no
// sanitizer.  With a GPU present the program does nothing: fake pointers must never reach a kernel.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "arctic_mi355x.h"

static std::mt19937_64 rng;
static int64_t pick(int64_t lo, int64_t hi) { return lo + (int64_t)(rng() % (uint64_t)(hi - lo + 1)); }
static int64_t size_like() {
  switch (pick(0, 9)) {
    case 0: return 0;
    case 1: return -pick(1, 5);
    case 2: return pick(1, 4);
    case 3: return (int64_t)1 << pick(5, 40);
    case 4: return INT64_MAX - pick(0, 3);
    case 5: return ((int64_t)1 << 31) - pick(0, 2);
    default: return pick(1, 5000);
  }
}
static int64_t plus(int64_t a, int64_t b) { return a > INT64_MAX - b ? INT64_MAX : a + b; }   // b >= 0
static int64_t times(int64_t a, int64_t b) {   // of non-negative numbers, saturating
  if (a < 0 || b < 0) return 0;
  return b != 0 && a > INT64_MAX / b ? INT64_MAX : a * b;
}
static int small_int() {
  switch (pick(0, 7)) {
    case 0: return 0;
    case 1: return -(int)pick(1, 3);
    case 2: return INT32_MAX;
    case 3: return (int)pick(1, 3) * 16;
    case 4: return 128;
    default: return (int)pick(1, 600);
  }
}
static void *dev_ptr() {
  switch (pick(0, 11)) {
    case 0: return nullptr;
    case 1: return (void *)(uintptr_t)(0x7f0000000000ull + (uint64_t)pick(1, 255));   // misaligned
    default: return (void *)(uintptr_t)(0x7f0000000000ull + (uint64_t)pick(0, 1 << 20) * 256);
  }
}
static int dtype_code() { return (int)pick(-1, 4); }

int main(int argc, char **argv) {
  int devices = 0;
  if (hipGetDeviceCount(&devices) == hipSuccess && devices > 0) {
    std::puts("skipped: a GPU is present");
    return 0;
  }
  rng.seed(argc > 1 ? (uint64_t)std::atoll(argv[1]) : 1u);
  const int calls = argc > 2 ? std::atoi(argv[2]) : 20000;
  long accepted = 0, rejected = 0, launched = 0;
  if (arctic_abi_version() != ARCTIC_ABI_VERSION) return 2;
  for (int it = 0; it < calls; ++it) {
    int rc = -1;
    const int which = (int)pick(0, 12);
    void *stream = nullptr;
    if (which <= 2) {
      int layers = pick(0, 3) == 0 ? small_int() : (int)pick(1, 80);
      const size_t entries = layers > 0 && layers <= 4096 ? (size_t)layers : 1;
      // heap tables of exactly `layers` entries: a read past the end is a sanitizer report
      std::vector<const void *> kc(entries), vc(entries);
      std::vector<const float *> ks(entries), vs(entries);
      for (size_t l = 0; l < entries; ++l) {
        kc[l] = dev_ptr(); vc[l] = dev_ptr(); ks[l] = (const float *)dev_ptr(); vs[l] = (const float *)dev_ptr();
      }
      const bool null_tables = pick(0, 15) == 0;
      const int heads = pick(0, 4) ? (int)pick(1, 16) : small_int(), head_size = pick(0, 4) ? (int)pick(1, 8) * 32 : small_int();
      const int block_size = pick(0, 4) ? 16 : small_int();
      const int64_t tokens = size_like(), n = times(heads, head_size);
      const int64_t stride = pick(0, 3) ? plus(times(n, layers > 0 && layers < 4096 ? layers : 1), pick(0, 1) * 8) : size_like();
      const int64_t block_stride = pick(0, 3) ? times(times(n, block_size), pick(1, 2)) : size_like();
      const int64_t blocks = pick(0, 2) ? pick(1, 1 << 20) : size_like();
      const int src = dtype_code(), kv = (int)pick(-1, 3);
      if (which == 0) {
        rc = arctic_reshape_and_cache_flash_bulk(dev_ptr(), dev_ptr(), stride, stride, null_tables ? nullptr : kc.data(),
                                                 vc.data(), ks.data(), vs.data(), (const int64_t *)dev_ptr(), tokens, layers,
                                                 heads, head_size, block_size, block_stride, blocks, src, kv, stream);
      } else {
        const int64_t nidx = size_like(), nsrc = pick(0, 2) ? plus(tokens, pick(0, 9)) : size_like();
        const int ib = pick(0, 5) ? (pick(0, 1) ? 8 : 4) : (int)pick(-1, 9);
        if (which == 1)
          rc = arctic_reshape_and_cache_flash_bulk_select(
              dev_ptr(), dev_ptr(), stride, stride, null_tables ? nullptr : kc.data(), vc.data(), ks.data(), vs.data(),
              (const int64_t *)dev_ptr(), tokens, layers, heads, head_size, block_size, block_stride, blocks, src, kv,
              (const int64_t *)dev_ptr(), dev_ptr(), ib, nidx, nsrc, dev_ptr(), dev_ptr(), stride, stride, stream);
        else
          rc = arctic_reshape_and_cache_flash_bulk_select_static(
              dev_ptr(), dev_ptr(), stride, stride, null_tables ? nullptr : kc.data(), vc.data(), ks.data(), vs.data(),
              (const int64_t *)dev_ptr(), tokens, layers, heads, head_size, block_size, block_stride, blocks, src, kv,
              dev_ptr(), ib, nidx, nsrc, dev_ptr(), dev_ptr(), stride, stride, stream);
      }
    } else if (which == 3) {
      rc = arctic_build_row_map((int64_t *)dev_ptr(), size_like(), dev_ptr(), (int)pick(-1, 9), size_like(), stream);
    } else if (which == 4) {
      const int heads = small_int(), head_size = pick(0, 3) ? (int)pick(1, 16) * 16 : small_int();
      rc = arctic_reshape_and_cache_flash_fp4(dev_ptr(), dev_ptr(), size_like(), size_like(), dev_ptr(), dev_ptr(), dev_ptr(),
                                              dev_ptr(), (const int64_t *)dev_ptr(), size_like(), heads, head_size,
                                              small_int(), size_like(), size_like(), size_like(), size_like(), dtype_code(),
                                              stream);
    } else if (which == 5) {
      rc = arctic_speculator_ln(dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), size_like(), small_int(), size_like(), 1e-6f,
                                dtype_code(), stream);
    } else if (which == 6) {
      rc = arctic_speculator_add_ln_act(dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), size_like(), small_int(),
                                        size_like(), size_like(), 1.5f, 1e-6f, (int)pick(-1, 4), 0.7f, dtype_code(), stream);
    } else if (which == 7) {
      rc = arctic_speculator_embed_add_ln_act(dev_ptr(), dev_ptr(), dev_ptr(), (const int64_t *)dev_ptr(), dev_ptr(), dev_ptr(),
                                              size_like(), small_int(), size_like(), size_like(), size_like(), 1.5f, 1e-6f,
                                              (int)pick(-1, 4), 0.7f, dtype_code(), stream);
    } else if (which == 8 || which == 9) {
      const int D = pick(0, 3) ? (int)pick(1, 64) * 64 : small_int();
      auto fn = which == 8 ? arctic_sum_lstm : arctic_sum_lstm_shared_z;
      rc = fn(dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), size_like(), D,
              pick(0, 2) ? 4 * (int64_t)D : size_like(), pick(0, 2) ? 4 * (int64_t)D : size_like(), size_like(),
              pick(0, 2) ? (int64_t)D : size_like(), 23.0f, 1e-6f, 1e-6f, (int)pick(0, 1), dtype_code(), stream);
    } else if (which == 10) {
      const int D = pick(0, 3) ? (int)pick(1, 64) * 64 : small_int();
      rc = arctic_sum_lstm_embedded(dev_ptr(), dev_ptr(), dev_ptr(), dev_ptr(), (const int64_t *)dev_ptr(), dev_ptr(), dev_ptr(),
                                    dev_ptr(), dev_ptr(), dev_ptr(), size_like(), D, size_like(), size_like(), size_like(),
                                    size_like(), size_like(), 23.0f, 1e-6f, 1e-6f, (int)pick(0, 1), dtype_code(), stream);
    } else if (which == 11) {
      const int nt = pick(0, 3) ? (int)pick(1, 8) : small_int();
      const size_t entries = nt > 0 && nt <= 4096 ? (size_t)nt : 1;
      std::vector<const void *> src(entries);
      std::vector<void *> dst(entries);
      std::vector<int64_t> rb(entries), ss(entries), ds(entries);
      for (size_t i = 0; i < entries; ++i) {
        src[i] = dev_ptr(); dst[i] = dev_ptr();
        rb[i] = pick(0, 3) ? pick(1, 1024) * 16 : size_like();
        ss[i] = pick(0, 3) ? plus(rb[i], pick(0, 2) * 16) : size_like();
        ds[i] = pick(0, 3) ? rb[i] : size_like();
      }
      rc = arctic_gather_rows(nt, pick(0, 15) ? src.data() : nullptr, dst.data(), rb.data(), ss.data(), ds.data(), dev_ptr(),
                              pick(0, 5) ? 8 : (int)pick(-1, 9), size_like(), size_like(), (int)pick(0, 1), stream);
    } else {
      rc = arctic_argmax_clamp((int64_t *)dev_ptr(), dev_ptr(), size_like(), small_int(), size_like(), size_like(), dtype_code(),
                               stream);
    }
    if (rc == ARCTIC_OK) {
      ++accepted;   // nothing to do (an empty batch, no layers)
    } else {
      ++rejected;
      launched += rc == ARCTIC_ERR_LAUNCH;
      if (rc != ARCTIC_ERR_INVALID_ARGUMENT && rc != ARCTIC_ERR_UNSUPPORTED && rc != ARCTIC_ERR_LAUNCH) {
        std::fprintf(stderr, "abi_host_fuzz: entry %d returned an unknown code %d (call %d)\n", which, rc, it);
        return 1;
      }
      const char *msg = arctic_last_error();
      if (!msg || !*msg) {
        std::fprintf(stderr, "abi_host_fuzz: entry %d failed with code %d and no message (call %d)\n", which, rc, it);
        return 1;
      }
    }
  }
  std::printf("ok %ld returned without work, %ld failed with a message, %ld of them at the launch\n", accepted, rejected,
              launched);
  return 0;
}
