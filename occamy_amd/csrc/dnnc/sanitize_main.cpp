// Driver of the sanitizer build of the host side (make asan): the ONNX reader, the pass pipeline, the planner and
// the executor, compiled with -fsanitize=address,undefined into one executable together with this file, are fed
// ONNX files and mutations of them.  (The reference runs its passes under whatever sanitizers an LLVM build is
// configured with; here the same job is one make target and one test.)
//
//   dnnc_sanitize model.onnx [more.onnx ...] [--mutations N] [--seed S] [--run ORACLE.so]
//
// Per file: the file as it is, then N mutations of it (truncated at a random byte, a few random bytes changed,
// a random run of bytes dropped or doubled, or several of these), each through dnncGraphFromOnnx and, when the
// reader accepts it, dnncCompile with the reference's flags and with every fusion; with --run, accepted programs
// also run once through the given host build of the runtime ABI on zero inputs.  A refusal is fine; what counts
// is that the process ends normally (the sanitizers abort on the first finding).  Exit status 0 and a line of
// counts, or the sanitizer's report.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../../include/dnnc.h"

static uint64_t g_state = 1;
static uint64_t rnd() {  // splitmix64
  uint64_t z = (g_state += 0x9e3779b97f4a7c15ull);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

static std::vector<uint8_t> mutate(const std::vector<uint8_t> &in) {
  std::vector<uint8_t> b = in;
  const int rounds = 1 + (int)(rnd() % 3);
  for (int r = 0; r < rounds && !b.empty(); r++) {
    switch (rnd() % 4) {
      case 0: b.resize((size_t)(rnd() % (b.size() + 1))); break;
      case 1:
        for (int i = 0, n = 1 + (int)(rnd() % 8); i < n && !b.empty(); i++) b[(size_t)(rnd() % b.size())] = (uint8_t)rnd();
        break;
      case 2: {
        const size_t at = (size_t)(rnd() % b.size()), n = std::min(b.size() - at, (size_t)(1 + rnd() % 64));
        b.erase(b.begin() + (long)at, b.begin() + (long)(at + n));
        break;
      }
      default: {
        const size_t at = (size_t)(rnd() % b.size()), n = std::min(b.size() - at, (size_t)(1 + rnd() % 64));
        const std::vector<uint8_t> run(b.begin() + (long)at, b.begin() + (long)(at + n));
        b.insert(b.begin() + (long)at, run.begin(), run.end());
        break;
      }
    }
  }
  return b;
}

struct Counts { long read = 0, accepted = 0, compiled = 0, ran = 0; };

static void one(const std::vector<uint8_t> &bytes, const char *runtime, Counts &c) {
  c.read++;
  dnncOptions plain{};
  plain.const_at_use = plain.dealloc_opt = plain.pool_opt = 1;
  dnncOptions fused = plain;
  fused.fusion = fused.fuse_residual = fused.fuse_activations = fused.recompose = fused.fuse_matmul_bias = 1;
  fused.fuse_attention = fused.fuse_first_layer_maxpool = fused.fuse_projection_shortcut = fused.alias_copies = 1;
  fused.inplace_residual = fused.compact_pool = 1;
  for (const dnncOptions *opt : {&plain, &fused}) {
    dnncGraph *g = dnncGraphFromOnnx(bytes.data(), (int64_t)bytes.size());  // a graph compiles once
    if (!g) return;
    if (opt == &plain) c.accepted++;
    dnncProgram *p = dnncCompile(g, opt);
    if (p) {
      c.compiled++;
      (void)dnncProgramText(p);
      (void)dnncProgramEvents(p, nullptr, nullptr, nullptr, nullptr, 0);
      // run it when it is small (a mutated shape can ask for any amount of memory)
      int64_t in_bytes = 0, out_bytes = 0;
      bool ok = dnncProgramPoolBytes(p) < (64ll << 20);
      std::vector<std::vector<uint8_t>> ins, outs;
      for (int32_t i = 0; ok && i < dnncGraphNumInputs(g); i++) {
        int32_t dt = 0, rank = 0;
        int64_t d[8];
        if (dnncGraphInputInfo(g, i, &dt, &rank, d, 8) || rank > 8) { ok = false; break; }
        int64_t n = dt == DNNC_F16 ? 2 : dt == DNNC_F32 ? 4 : 8;
        for (int32_t k = 0; k < rank; k++) n *= d[k];
        ok = n >= 0 && n < (64ll << 20);
        if (ok) { ins.emplace_back((size_t)n, 0); in_bytes += n; }
      }
      for (int32_t i = 0; ok && i < dnncProgramNumOutputs(p); i++) {
        int32_t dt = 0, rank = 0;
        int64_t d[8];
        if (dnncProgramOutputInfo(p, i, &dt, &rank, d)) { ok = false; break; }
        int64_t n = dt == DNNC_F16 ? 2 : dt == DNNC_F32 ? 4 : 8;
        for (int32_t k = 0; k < rank; k++) n *= d[k];
        ok = n >= 0 && n < (64ll << 20);
        if (ok) { outs.emplace_back((size_t)n + 8, 0); out_bytes += n; }
      }
      if (runtime && ok && in_bytes + out_bytes < (128ll << 20)) {
        for (int mode : {DNNC_MODE_OCCAMY, DNNC_MODE_RESIDENT}) {
          dnncSession *s = dnncSessionCreate(p, runtime, mode);
          if (!s) continue;
          std::vector<const void *> ip;
          std::vector<void *> op;
          for (auto &v : ins) ip.push_back(v.data());
          for (auto &v : outs) op.push_back(v.data());
          ip.push_back(nullptr);
          op.push_back(nullptr);
          if (dnncSessionRun(s, ip.data(), op.data()) == 0) c.ran++;
          dnncSessionDestroy(s);
        }
      }
      dnncProgramDestroy(p);
    }
    dnncGraphDestroy(g);
  }
}

int main(int argc, char **argv) {
  std::vector<std::string> files;
  long mutations = 200;
  const char *runtime = nullptr;
  for (int i = 1; i < argc; i++) {
    if (!strcmp(argv[i], "--mutations") && i + 1 < argc) mutations = atol(argv[++i]);
    else if (!strcmp(argv[i], "--seed") && i + 1 < argc) g_state = (uint64_t)atoll(argv[++i]);
    else if (!strcmp(argv[i], "--run") && i + 1 < argc) runtime = argv[++i];
    else files.push_back(argv[i]);
  }
  if (files.empty()) { fprintf(stderr, "usage: dnnc_sanitize model.onnx [...] [--mutations N] [--seed S] [--run ORACLE.so]\n"); return 2; }
  Counts c;
  for (const std::string &f : files) {
    FILE *fp = fopen(f.c_str(), "rb");
    if (!fp) { fprintf(stderr, "cannot open %s\n", f.c_str()); return 2; }
    std::vector<uint8_t> bytes;
    uint8_t buf[65536];
    size_t n;
    while ((n = fread(buf, 1, sizeof buf, fp)) > 0) bytes.insert(bytes.end(), buf, buf + n);
    fclose(fp);
    one(bytes, runtime, c);
    if (c.accepted == 0) { fprintf(stderr, "%s: the unmodified file was refused: %s\n", f.c_str(), dnncLastError()); return 3; }
    for (long m = 0; m < mutations; m++) one(mutate(bytes), runtime, c);
  }
  printf("inputs %ld, accepted by the reader %ld, compiled %ld (of two flag sets each), ran %ld\n", c.read, c.accepted, c.compiled, c.ran);
  return 0;
}
