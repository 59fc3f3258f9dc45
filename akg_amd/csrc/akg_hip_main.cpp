/**
 * akg-hip: command-line driver over the C ABI. One tool where the reference has four
 * (mindspore-translate, akg-opt, akg-translate, akg-ptx-replace; akg-mlir/tools), because there is one
 * step here: op description in, gfx950 code object + meta out.
 *
 *   akg-hip translate X.info            print the typed op graph (mindspore-translate -json-to-mindspore)
 *   akg-hip emit X.info                 print the emitted HIP source
 *   akg-hip compile X.info -o DIR       write <op>.hsaco, <op>.json, <op>_shape_arg.txt, <op>.hip to DIR
 *   akg-hip info X.info                 print signature, family, launch shape, algorithmic bytes
 *   ... --shapes "32,1,48,48;32,12,48,48"   with emit / compile / info / run: X.info is a dynamic-shape description (-1
 *                                       extents); it is specialised to these input shapes (one per input, in
 *                                       input_desc order) through akg_hip_dynamic_specialize first
 *   akg-hip run X.info [-n N] [-r R] [--inputs DIR] [--dump DIR] [--expect DIR]
 *                                       what `akg_benchmark -e gpu -f X.info -p` does (benchmark.py:94-130): seeded
 *                                       inputs, NaN-prefilled outputs, one call on host buffers, then R x N timed
 *                                       launches on device buffers; prints the time, the achieved bandwidth, the
 *                                       outputs' checksums and how many NaNs they hold.
 *                                       The numeric compare of the reference's tool is split from the expectation's
 *                                       maker, so that this binary links no CPU implementation of the operators:
 *                                       --dump writes every argument as DIR/arg<i>.bin (raw little-endian elements,
 *                                       inputs as given, outputs as computed), --inputs reads the inputs from such
 *                                       files, --expect compares each output with DIR/arg<i>.bin (integers and bool
 *                                       bit for bit; float32 within rtol 1e-5, float16 / bfloat16 within rtol 1e-2 and
 *                                       atol 1e-3, float64 within rtol 1e-12; a NaN matches a NaN) and exits 1 on a
 *                                       mismatch.
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
               "       akg-hip run X.info [-n launches per measurement] [-r measurements]\n"
               "                          [--inputs DIR] [--dump DIR] [--expect DIR]\n"
               "       emit / compile / info / run take --shapes \"d,d,..;d,d,..\" for a dynamic-shape description\n");
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

std::string argPath(const char *dir, int i) { return std::string(dir) + "/arg" + std::to_string(i) + ".bin"; }

bool writeAll(const std::string &path, const std::vector<unsigned char> &bytes) {
  std::ofstream f(path, std::ios::binary);
  f.write(reinterpret_cast<const char *>(bytes.data()), static_cast<std::streamsize>(bytes.size()));
  return static_cast<bool>(f);
}

float halfValue(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  const int exp = (h >> 10) & 0x1F;
  const uint32_t man = h & 0x3FFu;
  float f;
  if (exp == 0) {
    f = static_cast<float>(man) * 0x1p-24f;   // subnormal or zero
    uint32_t u;
    std::memcpy(&u, &f, 4);
    u |= sign;
    std::memcpy(&f, &u, 4);
    return f;
  }
  const uint32_t u = sign | (exp == 31 ? 0x7F800000u : static_cast<uint32_t>(exp - 15 + 127) << 23) | (man << 13);
  std::memcpy(&f, &u, 4);
  return f;
}

// Element `i` of a float tensor as a double (float16 / bfloat16 / float32 / float64).
double floatAt(const char *t, const unsigned char *base, size_t i) {
  if (std::strcmp(t, "float64") == 0) {
    double v;
    std::memcpy(&v, base + i * 8, 8);
    return v;
  }
  if (std::strcmp(t, "float32") == 0) {
    float v;
    std::memcpy(&v, base + i * 4, 4);
    return v;
  }
  uint16_t h;
  std::memcpy(&h, base + i * 2, 2);
  if (std::strcmp(t, "float16") == 0) return halfValue(h);
  const uint32_t u = static_cast<uint32_t>(h) << 16;
  float v;
  std::memcpy(&v, &u, 4);
  return v;
}

// How many elements of output `d` differ from the expectation by more than the type's tolerance; the
// first one is described in *first. Integers and bool compare bit for bit.
long long countMismatches(const akg_hip_tensor_desc &d, const std::vector<unsigned char> &got,
                          const std::vector<unsigned char> &want, std::string *first) {
  const char *t = dtypeName(d.dtype);
  const bool isFloat = std::strncmp(t, "float", 5) == 0 || std::strcmp(t, "bfloat16") == 0;
  const size_t esize = std::strstr(t, "64") ? 8 : std::strstr(t, "32") ? 4 : std::strstr(t, "16") ? 2 : 1;
  const size_t n = got.size() / esize;
  long long bad = 0;
  for (size_t i = 0; i < n; ++i) {
    bool same;
    char what[160];
    if (isFloat) {
      const double a = floatAt(t, got.data(), i), b = floatAt(t, want.data(), i);
      const double rtol = esize == 2 ? 1e-2 : esize == 4 ? 1e-5 : 1e-12, atol = esize == 2 ? 1e-3 : 0.0;
      const double mag = b < 0 ? -b : b, diff = a > b ? a - b : b - a;
      same = (a != a && b != b) || a == b || diff <= atol + rtol * mag;
      if (!same) std::snprintf(what, sizeof what, "element %zu: got %.9g, expected %.9g", i, a, b);
    } else {
      same = std::memcmp(got.data() + i * esize, want.data() + i * esize, esize) == 0;
      if (!same) {
        int64_t a = 0, b = 0;
        std::memcpy(&a, got.data() + i * esize, esize);
        std::memcpy(&b, want.data() + i * esize, esize);
        std::snprintf(what, sizeof what, "element %zu: got 0x%llx, expected 0x%llx", i,
                      static_cast<unsigned long long>(a), static_cast<unsigned long long>(b));
      }
    }
    if (!same && bad++ == 0) *first = what;
  }
  return bad;
}

int runKernel(akg_hip_kernel_t *k, int number, int repeat, const char *inputsDir, const char *dumpDir,
              const char *expectDir) {
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
    } else if (inputsDir != nullptr) {
      std::string raw;
      if (!readAll(argPath(inputsDir, i).c_str(), &raw) || static_cast<int64_t>(raw.size()) != d.bytes) {
        std::fprintf(stderr, "akg-hip: %s must hold the %lld bytes of input %s\n", argPath(inputsDir, i).c_str(),
                     static_cast<long long>(d.bytes), d.name);
        return 1;
      }
      host[static_cast<size_t>(i)].assign(raw.begin(), raw.end());
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
  if (dumpDir != nullptr) {
    for (int i = 0; i < n; ++i) {
      if (!writeAll(argPath(dumpDir, i), host[static_cast<size_t>(i)])) {
        std::fprintf(stderr, "akg-hip: cannot write %s\n", argPath(dumpDir, i).c_str());
        return 1;
      }
    }
  }
  int status = 0;
  if (expectDir != nullptr) {
    for (int i = 0; i < n; ++i) {
      const akg_hip_tensor_desc &d = descs[static_cast<size_t>(i)];
      if (!d.is_output) continue;
      std::string raw, first;
      if (!readAll(argPath(expectDir, i).c_str(), &raw) || static_cast<int64_t>(raw.size()) != d.bytes) {
        std::fprintf(stderr, "akg-hip: %s must hold the %lld bytes expected of output %s\n",
                     argPath(expectDir, i).c_str(), static_cast<long long>(d.bytes), d.name);
        return 1;
      }
      const std::vector<unsigned char> want(raw.begin(), raw.end());
      const long long bad = countMismatches(d, host[static_cast<size_t>(i)], want, &first);
      if (bad == 0) {
        std::printf("compare %-12s ok\n", d.name);
      } else {
        std::printf("compare %-12s MISMATCH in %lld elements, first %s\n", d.name, bad, first.c_str());
        status = 1;
      }
    }
  }
  return status;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc < 3) return usage();
  const std::string cmd = argv[1];
  const char *path = argv[2];
  const char *outDir = nullptr, *inputsDir = nullptr, *dumpDir = nullptr, *expectDir = nullptr, *shapesText = nullptr;
  int number = 10, repeat = 5;
  for (int i = 3; i + 1 < argc; ++i) {
    if (std::strcmp(argv[i], "--inputs") == 0) inputsDir = argv[i + 1];
    if (std::strcmp(argv[i], "--dump") == 0) dumpDir = argv[i + 1];
    if (std::strcmp(argv[i], "--expect") == 0) expectDir = argv[i + 1];
    if (std::strcmp(argv[i], "--shapes") == 0) shapesText = argv[i + 1];
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
  akg_hip_dynamic_t *dyn = nullptr;   // owns k when the description is a dynamic one
  int rc;
  if (shapesText != nullptr) {
    std::string text;
    if (!readAll(path, &text)) {
      std::fprintf(stderr, "akg-hip: cannot read %s\n", path);
      return 1;
    }
    std::vector<std::vector<int64_t>> shapes(1);
    for (const char *p = shapesText; *p != 0; ++p) {
      if (*p == ';') {
        shapes.emplace_back();
      } else if (*p >= '0' && *p <= '9') {
        char *end = nullptr;
        shapes.back().push_back(std::strtoll(p, &end, 10));
        p = end - 1;
      } else if (*p != ',' && *p != ' ') {
        std::fprintf(stderr, "akg-hip: --shapes takes extents separated by ',' and shapes separated by ';'\n");
        return 2;
      }
    }
    std::vector<const int64_t *> shapePtrs;
    std::vector<int32_t> ranks;
    for (const auto &sh : shapes) {
      shapePtrs.push_back(sh.data());
      ranks.push_back(static_cast<int32_t>(sh.size()));
    }
    rc = akg_hip_dynamic_create(text.data(), text.size(), cmd == "compile" ? outDir : nullptr, &dyn);
    if (rc == AKG_HIP_OK) rc = akg_hip_dynamic_specialize(dyn, shapePtrs.data(), ranks.data(), static_cast<int>(shapes.size()), &k);
  } else {
    rc = akg_hip_compile_file(path, cmd == "compile" ? outDir : nullptr, &k);
  }
  if (rc != AKG_HIP_OK) {
    std::fprintf(stderr, "akg-hip: error %d: %s\n", rc, akg_hip_last_error());
    if (dyn) akg_hip_dynamic_destroy(dyn);
    return 1;
  }
  int status = 0;
  if (cmd == "run") {
    status = runKernel(k, number, repeat, inputsDir, dumpDir, expectDir);
  } else if (cmd == "emit") {
    const char *src = nullptr;
    akg_hip_kernel_source(k, &src);
    std::fputs(src, stdout);
  } else {
    printInfo(k);
  }
  if (dyn) {
    akg_hip_dynamic_destroy(dyn);
  } else {
    akg_hip_kernel_destroy(k);
  }
  return status;
}
