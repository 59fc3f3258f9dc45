/**
 * akg-hip: command-line driver over the C ABI. One tool where the reference has four
 * (mindspore-translate, akg-opt, akg-translate, akg-ptx-replace; akg-mlir/tools), because there is one
 * step here: op description in, gfx950 code object + meta out.
 *
 *   akg-hip translate X.info            print the typed op graph (mindspore-translate -json-to-mindspore)
 *   akg-hip emit X.info                 print the emitted HIP source
 *   akg-hip compile X.info -o DIR       write <op>.hsaco, <op>.json, <op>_shape_arg.txt, <op>.hip to DIR
 *   akg-hip info X.info                 print signature, family, launch shape, algorithmic bytes
 *   akg-hip run X.info [-n N] [-r R]    what `akg_benchmark -e gpu -f X.info -p` does without the numeric compare
 *                                       (benchmark.py:94-130): seeded inputs, NaN-prefilled outputs, one call on host
 *                                       buffers, then R x N timed launches on device buffers; prints the time, the
 *                                       achieved bandwidth, the outputs' checksums and how many NaNs they hold
 */
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "../../include/akg_hip.h"

namespace {

int usage() {
  std::fprintf(stderr,
               "usage: akg-hip translate X.info\n"
               "       akg-hip emit X.info\n"
               "       akg-hip compile X.info -o DIR\n"
               "       akg-hip info X.info\n"
               "       akg-hip run X.info [-n launches per measurement] [-r measurements]\n");
  return 2;
}

bool readAll(const char *path, std::string *out) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return false;
  std::ostringstream ss;
  ss << f.rdbuf();
  *out = ss.str();
  return true;
}

const char *dtypeName(int d) {
  static const char *const names[] = {"bool",    "int8",     "int16",   "int32",  "int64",
                                      "float16", "bfloat16", "float32", "float64"};
  return (d >= 0 && d < 9) ? names[d] : "?";
}

void printInfo(akg_hip_kernel_t *k) {
  akg_hip_kernel_info info;
  if (akg_hip_kernel_get_info(k, &info) != AKG_HIP_OK) return;
  std::printf("kernel      %s\n", info.kernel_name);
  std::printf("family      %s (fusion class %s)\n", info.family, info.operator_type);
  std::printf("grid        %u x %u x %u\n", info.grid[0], info.grid[1], info.grid[2]);
  std::printf("block       %u x %u x %u\n", info.block[0], info.block[1], info.block[2]);
  std::printf("alg. bytes  %llu\n", static_cast<unsigned long long>(info.algorithmic_bytes));
  std::printf("alg. ops    %llu\n", static_cast<unsigned long long>(info.algorithmic_ops));
  std::printf("cache hit   %d\n", info.cache_hit);
  int n = 0;
  akg_hip_kernel_num_tensors(k, &n);
  for (int i = 0; i < n; ++i) {
    akg_hip_tensor_desc d;
    if (akg_hip_kernel_tensor(k, i, &d) != AKG_HIP_OK) continue;
    std::printf("arg %d  %-6s %-12s %-9s [", i, d.is_output ? "output" : "input", d.name, dtypeName(d.dtype));
    for (int r = 0; r < d.rank; ++r) std::printf("%s%lld", r ? "," : "", static_cast<long long>(d.shape[r]));
    std::printf("]  %lld bytes\n", static_cast<long long>(d.bytes));
  }
}

// float -> IEEE half bits, round to nearest even, for |f| < 2 (what fillInput makes).
uint16_t halfBits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  const uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
  const int exp = static_cast<int>((u >> 23) & 0xFFu) - 127 + 15;
  uint32_t man = u & 0x7FFFFFu;
  if (exp <= 0) {                       // subnormal half or zero
    if (exp < -10) return sign;
    man |= 0x800000u;
    const int shift = 14 - exp;
    const uint32_t q = man >> shift, rest = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
    return static_cast<uint16_t>(sign | (q + ((rest > half || (rest == half && (q & 1u))) ? 1u : 0u)));
  }
  const uint32_t q = (static_cast<uint32_t>(exp) << 10) | (man >> 13), rest = man & 0x1FFFu;
  return static_cast<uint16_t>(sign | (q + ((rest > 0x1000u || (rest == 0x1000u && (q & 1u))) ? 1u : 0u)));
}

// Seeded values of tensor `d`: floats uniform in [-1, 1), integers in [0, 1000), bool 0 / 1.
void fillInput(const akg_hip_tensor_desc &d, uint64_t seed, std::vector<unsigned char> *bytes) {
  bytes->assign(static_cast<size_t>(d.bytes), 0);
  uint64_t x = seed * 0x9E3779B97F4A7C15ull + 0x1234567ull;
  auto next = [&x]() {
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    return x;
  };
  const char *t = dtypeName(d.dtype);
  const size_t esize = std::strstr(t, "64") ? 8 : std::strstr(t, "32") ? 4 : std::strstr(t, "16") ? 2 : 1;
  const size_t n = bytes->size() / esize;
  for (size_t i = 0; i < n; ++i) {
    const uint64_t r = next();
    const float f = static_cast<float>(static_cast<double>(r >> 11) / 9007199254740992.0 * 2.0 - 1.0);
    unsigned char *p = bytes->data() + i * esize;
    if (std::strcmp(t, "float32") == 0) {
      std::memcpy(p, &f, 4);
    } else if (std::strcmp(t, "float64") == 0) {
      const double v = f;
      std::memcpy(p, &v, 8);
    } else if (std::strcmp(t, "bfloat16") == 0) {
      uint32_t u;
      std::memcpy(&u, &f, 4);
      const uint16_t h = static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
      std::memcpy(p, &h, 2);
    } else if (std::strcmp(t, "float16") == 0) {
      const uint16_t h = halfBits(f);
      std::memcpy(p, &h, 2);
    } else if (std::strcmp(t, "bool") == 0) {
      *p = static_cast<unsigned char>(r & 1u);
    } else {
      const int64_t v = static_cast<int64_t>(r % 1000u);
      std::memcpy(p, &v, esize);   // little endian: the low bytes
    }
  }
}

// NaNs left in a float output (elements the kernel failed to write, or produced), -1 for other types.
long long countNans(const akg_hip_tensor_desc &d, const std::vector<unsigned char> &bytes) {
  const char *t = dtypeName(d.dtype);
  long long nans = 0;
  if (std::strcmp(t, "float32") == 0) {
    for (size_t i = 0; i + 4 <= bytes.size(); i += 4) {
      uint32_t u;
      std::memcpy(&u, bytes.data() + i, 4);
      nans += (u & 0x7FFFFFFFu) > 0x7F800000u;
    }
  } else if (std::strcmp(t, "float16") == 0 || std::strcmp(t, "bfloat16") == 0) {
    const uint16_t expMask = std::strcmp(t, "float16") == 0 ? 0x7C00u : 0x7F80u;
    for (size_t i = 0; i + 2 <= bytes.size(); i += 2) {
      uint16_t u;
      std::memcpy(&u, bytes.data() + i, 2);
      nans += (u & 0x7FFFu) > expMask;
    }
  } else {
    return -1;
  }
  return nans;
}

int runKernel(akg_hip_kernel_t *k, int number, int repeat) {
  akg_hip_kernel_info info;
  int n = 0;
  if (akg_hip_kernel_get_info(k, &info) != AKG_HIP_OK || akg_hip_kernel_num_tensors(k, &n) != AKG_HIP_OK) return 1;
  std::vector<akg_hip_tensor_desc> descs(static_cast<size_t>(n));
  std::vector<std::vector<unsigned char>> host(static_cast<size_t>(n));
  std::vector<void *> hostPtrs(static_cast<size_t>(n)), devPtrs(static_cast<size_t>(n), nullptr);
  for (int i = 0; i < n; ++i) {
    if (akg_hip_kernel_tensor(k, i, &descs[static_cast<size_t>(i)]) != AKG_HIP_OK) return 1;
    const akg_hip_tensor_desc &d = descs[static_cast<size_t>(i)];
    if (d.is_output) {
      host[static_cast<size_t>(i)].assign(static_cast<size_t>(d.bytes), 0xFF);   // all-ones is a NaN in every float type
    } else {
      fillInput(d, 20260000ull + static_cast<uint64_t>(i), &host[static_cast<size_t>(i)]);
    }
    hostPtrs[static_cast<size_t>(i)] = host[static_cast<size_t>(i)].data();
  }
  int rc = akg_hip_run_host(k, hostPtrs.data(), n);
  if (rc != AKG_HIP_OK) {
    std::fprintf(stderr, "akg-hip: error %d: %s\n", rc, akg_hip_last_error());
    return 1;
  }
  bool ok = true;
  for (int i = 0; i < n && ok; ++i) {
    const size_t bytes = host[static_cast<size_t>(i)].size();
    ok = hipMalloc(&devPtrs[static_cast<size_t>(i)], bytes ? bytes : 1) == hipSuccess &&
         hipMemcpy(devPtrs[static_cast<size_t>(i)], host[static_cast<size_t>(i)].data(), bytes, hipMemcpyHostToDevice) == hipSuccess;
  }
  double avgMs = 0.0;
  if (ok) {
    rc = akg_hip_profile(k, devPtrs.data(), n, number, repeat, &avgMs);
    if (rc != AKG_HIP_OK) std::fprintf(stderr, "akg-hip: error %d: %s\n", rc, akg_hip_last_error());
    ok = rc == AKG_HIP_OK;
  } else {
    std::fprintf(stderr, "akg-hip: cannot allocate device buffers\n");
  }
  for (void *p : devPtrs) {
    if (p) (void)hipFree(p);
  }
  if (!ok) return 1;
  std::printf("kernel      %s (%s)\n", info.kernel_name, info.family);
  std::printf("time        %.4f ms per launch (%d x %d launches)\n", avgMs, repeat, number);
  std::printf("bandwidth   %.1f GB/s on %llu algorithmic bytes\n",
              static_cast<double>(info.algorithmic_bytes) / (avgMs * 1e-3) / 1e9,
              static_cast<unsigned long long>(info.algorithmic_bytes));
  for (int i = 0; i < n; ++i) {
    const akg_hip_tensor_desc &d = descs[static_cast<size_t>(i)];
    if (!d.is_output) continue;
    uint64_t h = 1469598103934665603ull;   // FNV-1a over the bytes the host call returned
    for (unsigned char c : host[static_cast<size_t>(i)]) h = (h ^ c) * 1099511628211ull;
    std::printf("output %-12s %-9s fnv1a %016llx  nans %lld\n", d.name, dtypeName(d.dtype),
                static_cast<unsigned long long>(h), countNans(d, host[static_cast<size_t>(i)]));
  }
  return 0;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc < 3) return usage();
  const std::string cmd = argv[1];
  const char *path = argv[2];
  const char *outDir = nullptr;
  int number = 10, repeat = 5;
  for (int i = 3; i + 1 < argc; ++i) {
    if (std::strcmp(argv[i], "-o") == 0) outDir = argv[i + 1];
    if (std::strcmp(argv[i], "-n") == 0) number = std::atoi(argv[i + 1]);
    if (std::strcmp(argv[i], "-r") == 0) repeat = std::atoi(argv[i + 1]);
  }
  if (cmd == "translate") {
    std::string text;
    if (!readAll(path, &text)) {
      std::fprintf(stderr, "akg-hip: cannot read %s\n", path);
      return 1;
    }
    char *out = nullptr;
    if (akg_hip_translate(text.data(), text.size(), &out) != AKG_HIP_OK) {
      std::fprintf(stderr, "akg-hip: %s\n", akg_hip_last_error());
      return 1;
    }
    std::fputs(out, stdout);
    akg_hip_free_string(out);
    return 0;
  }
  if (cmd != "emit" && cmd != "compile" && cmd != "info" && cmd != "run") return usage();
  if (cmd == "compile" && outDir == nullptr) return usage();
  akg_hip_kernel_t *k = nullptr;
  int rc = akg_hip_compile_file(path, cmd == "compile" ? outDir : nullptr, &k);
  if (rc != AKG_HIP_OK) {
    std::fprintf(stderr, "akg-hip: error %d: %s\n", rc, akg_hip_last_error());
    return 1;
  }
  if (cmd == "run") {
    rc = runKernel(k, number, repeat);
    akg_hip_kernel_destroy(k);
    return rc;
  }
  if (cmd == "emit") {
    const char *src = nullptr;
    akg_hip_kernel_source(k, &src);
    std::fputs(src, stdout);
  } else {
    printInfo(k);
  }
  akg_hip_kernel_destroy(k);
  return 0;
}
