/**
 * akg-hip: command-line driver over the C ABI. One tool where the reference has four
 * (mindspore-translate, akg-opt, akg-translate, akg-ptx-replace; akg-mlir/tools), because there is one
 * step here: op description in, gfx950 code object + meta out.
 *
 *   akg-hip translate X.info            print the typed op graph (mindspore-translate -json-to-mindspore)
 *   akg-hip emit X.info                 print the emitted HIP source
 *   akg-hip compile X.info -o DIR       write <op>.hsaco, <op>.json, <op>_shape_arg.txt, <op>.hip to DIR
 *   akg-hip info X.info                 print signature, family, launch shape, algorithmic bytes
 */
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>

#include "../../include/akg_hip.h"

namespace {

int usage() {
  std::fprintf(stderr,
               "usage: akg-hip translate X.info\n"
               "       akg-hip emit X.info\n"
               "       akg-hip compile X.info -o DIR\n"
               "       akg-hip info X.info\n");
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

}  // namespace

int main(int argc, char **argv) {
  if (argc < 3) return usage();
  const std::string cmd = argv[1];
  const char *path = argv[2];
  const char *outDir = nullptr;
  for (int i = 3; i + 1 < argc; ++i) {
    if (std::strcmp(argv[i], "-o") == 0) outDir = argv[i + 1];
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
  if (cmd != "emit" && cmd != "compile" && cmd != "info") return usage();
  if (cmd == "compile" && outDir == nullptr) return usage();
  akg_hip_kernel_t *k = nullptr;
  int rc = akg_hip_compile_file(path, cmd == "compile" ? outDir : nullptr, &k);
  if (rc != AKG_HIP_OK) {
    std::fprintf(stderr, "akg-hip: error %d: %s\n", rc, akg_hip_last_error());
    return 1;
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
