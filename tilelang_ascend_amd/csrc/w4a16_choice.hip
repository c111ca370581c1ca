// Tuned kernel choice for the W4A16 operator: a process-wide table (M, N, K, group, in_dtype) -> kernel family that
// tlq_gemm_w4a16 / tlq_gemm_w4a16_ws consult before their own rules when called with TLQ_ALGO_AUTO.  The reference searches
// its configurations per call signature and keeps the winner (tilelang/autotuner/tuner.py:102-760, on disk through
// tilelang/cache/tuner_cache.py); here the kernels are pre-built, so what a search finds is WHICH of them runs, and this
// table is where the result lives for callers of the C ABI.  Host code only.
#include <atomic>
#include <mutex>
#include <shared_mutex>
#include <unordered_map>

#include "tlq_common.h"

namespace tlq {

namespace {

struct ChoiceKey {
  int64_t M, N, K, group;
  int in_dtype;
  bool operator==(const ChoiceKey& o) const { return M == o.M && N == o.N && K == o.K && group == o.group && in_dtype == o.in_dtype; }
};
struct ChoiceHash {
  size_t operator()(const ChoiceKey& k) const {
    uint64_t h = 0x9e3779b97f4a7c15ull;
    for (uint64_t v : {(uint64_t)k.M, (uint64_t)k.N, (uint64_t)k.K, (uint64_t)k.group, (uint64_t)k.in_dtype}) {
      h ^= v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
    }
    return (size_t)h;
  }
};

std::shared_mutex g_choice_lock;
std::unordered_map<ChoiceKey, int, ChoiceHash>& choice_table() {
  static std::unordered_map<ChoiceKey, int, ChoiceHash> t;
  return t;
}
std::atomic<int64_t> g_choice_count{0};  // entries in the table: the launch path looks nothing up while it is 0

bool valid_algo(int algo) { return algo >= TLQ_ALGO_AUTO && algo <= TLQ_ALGO_PANELM; }

}  // namespace

// The tuned family for this call signature, or TLQ_ALGO_AUTO.
int w4a16_choice_lookup(int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype) {
  if (g_choice_count.load(std::memory_order_acquire) == 0) return TLQ_ALGO_AUTO;
  std::shared_lock<std::shared_mutex> lk(g_choice_lock);
  const auto& t = choice_table();
  const auto it = t.find(ChoiceKey{M, N, K, group, in_dtype});
  return it == t.end() ? TLQ_ALGO_AUTO : it->second;
}

// Calls fn(algo) for every entry with this (M, N, K), whatever its group and type (workspace sizing).
void w4a16_choice_for_shape(int64_t M, int64_t N, int64_t K, void (*fn)(int algo, void* ctx), void* ctx) {
  if (g_choice_count.load(std::memory_order_acquire) == 0) return;
  std::shared_lock<std::shared_mutex> lk(g_choice_lock);
  for (const auto& kv : choice_table())
    if (kv.first.M == M && kv.first.N == N && kv.first.K == K) fn(kv.second, ctx);
}

}  // namespace tlq

extern "C" {

int tlq_w4a16_choice_set(int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype, int algo) {
  using namespace tlq;
  TLQ_REQUIRE(M >= 1 && N >= 1 && K >= 1 && group >= 1, "tlq_w4a16_choice_set: M, N, K and group must be positive (got %lld %lld %lld %lld)",
              (long long)M, (long long)N, (long long)K, (long long)group);
  TLQ_REQUIRE(in_dtype == TLQ_F16 || in_dtype == TLQ_BF16, "tlq_w4a16_choice_set: in_dtype must be float16 or bfloat16 (got %d)", in_dtype);
  TLQ_REQUIRE(valid_algo(algo), "tlq_w4a16_choice_set: bad algo %d", algo);
  std::unique_lock<std::shared_mutex> lk(g_choice_lock);
  auto& t = choice_table();
  const ChoiceKey key{M, N, K, group, in_dtype};
  if (algo == TLQ_ALGO_AUTO)
    t.erase(key);
  else
    t[key] = algo;
  g_choice_count.store((int64_t)t.size(), std::memory_order_release);
  return 0;
}

int tlq_w4a16_choice_get(int64_t M, int64_t N, int64_t K, int64_t group, int in_dtype) {
  return tlq::w4a16_choice_lookup(M, N, K, group, in_dtype);
}

void tlq_w4a16_choice_clear(void) {
  using namespace tlq;
  std::unique_lock<std::shared_mutex> lk(g_choice_lock);
  choice_table().clear();
  g_choice_count.store(0, std::memory_order_release);
}

int64_t tlq_w4a16_choice_count(void) { return tlq::g_choice_count.load(std::memory_order_acquire); }

// One entry per line: "M N K group in_dtype algo" (decimal; in_dtype and algo are the codes of tlq.h); '#' starts a comment.
int tlq_w4a16_choice_save(const char* path) {
  using namespace tlq;
  TLQ_REQUIRE(path && path[0], "tlq_w4a16_choice_save: no path");
  FILE* f = fopen(path, "w");
  TLQ_REQUIRE(f != nullptr, "tlq_w4a16_choice_save: cannot write %s", path);
  fprintf(f, "# libtlq W4A16 kernel choices: M N K group in_dtype algo (ABI version %d)\n", TLQ_ABI_VERSION);
  {
    std::shared_lock<std::shared_mutex> lk(g_choice_lock);
    for (const auto& kv : choice_table())
      fprintf(f, "%lld %lld %lld %lld %d %d\n", (long long)kv.first.M, (long long)kv.first.N, (long long)kv.first.K,
              (long long)kv.first.group, kv.first.in_dtype, kv.second);
  }
  const bool bad = ferror(f) != 0;
  const bool closed = fclose(f) == 0;
  TLQ_REQUIRE(!bad && closed, "tlq_w4a16_choice_save: write to %s failed", path);
  return 0;
}

// Adds the file's entries to the table (an entry for a signature already present replaces it).  A malformed line is an
// error and leaves the table as it was before the call.
int tlq_w4a16_choice_load(const char* path) {
  using namespace tlq;
  TLQ_REQUIRE(path && path[0], "tlq_w4a16_choice_load: no path");
  FILE* f = fopen(path, "r");
  TLQ_REQUIRE(f != nullptr, "tlq_w4a16_choice_load: cannot read %s", path);
  std::unordered_map<ChoiceKey, int, ChoiceHash> incoming;
  char line[256];
  int lineno = 0;
  bool ok = true;
  while (ok && fgets(line, sizeof(line), f)) {
    ++lineno;
    const char* p = line;
    while (*p == ' ' || *p == '\t') ++p;
    if (*p == '#' || *p == '\n' || *p == '\r' || *p == 0) continue;
    long long m, n, k, g;
    int dt, algo;
    char extra;
    const int got = sscanf(p, "%lld %lld %lld %lld %d %d %c", &m, &n, &k, &g, &dt, &algo, &extra);
    if (got != 6 || m < 1 || n < 1 || k < 1 || g < 1 || (dt != TLQ_F16 && dt != TLQ_BF16) || !valid_algo(algo) || algo == TLQ_ALGO_AUTO) {
      ok = false;
      break;
    }
    incoming[ChoiceKey{m, n, k, g, dt}] = algo;
  }
  fclose(f);
  TLQ_REQUIRE(ok, "tlq_w4a16_choice_load: %s line %d is not \"M N K group in_dtype algo\"", path, lineno);
  std::unique_lock<std::shared_mutex> lk(g_choice_lock);
  auto& t = choice_table();
  for (const auto& kv : incoming) t[kv.first] = kv.second;
  g_choice_count.store((int64_t)t.size(), std::memory_order_release);
  return 0;
}

}  // extern "C"
