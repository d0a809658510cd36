// libroller_hip.so -- host side of the Roller fp32 GEMM path on MI355X: hiprtc JIT of the kernel
// template, a code-object cache (in process and on disk), module load / launch, and the small
// set of memory, stream and event calls a benchmark needs.  Declarations and the reference
// calls they replace: include/roller_hip.h.
//
// Host-only translation unit (no device code): the kernel template is pulled in as text with
// .incbin and handed to hiprtc at run time.

#include "roller_hip.h"
#include "roller_scratch.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <shared_mutex>
#include <string>
#include <vector>

#if !defined(RL_TEMPLATE_PATH) || !defined(RL_SK_DECODE_PATH)
#error "build with -DRL_TEMPLATE_PATH=\"<path to gemm_f32_mfma.hip>\" -DRL_SK_DECODE_PATH=\"<path to gemm_sk_decode.inc>\""
#endif

// The kernel template and the work decomposition it includes, byte for byte, NUL-terminated.  The
// decomposition is also compiled into this file: the host fills the launch parameters with the
// same arithmetic that the workgroups decode them with.
__asm__(
    ".section .rodata\n"
    ".global rl_gemm_template_begin\n"
    "rl_gemm_template_begin:\n"
    ".incbin \"" RL_TEMPLATE_PATH "\"\n"
    ".byte 0\n"
    ".global rl_gemm_sk_decode_begin\n"
    "rl_gemm_sk_decode_begin:\n"
    ".incbin \"" RL_SK_DECODE_PATH "\"\n"
    ".byte 0\n"
    ".previous\n");
extern "C" const char rl_gemm_template_begin[];
extern "C" const char rl_gemm_sk_decode_begin[];

#include "gemm_sk_decode.inc"

namespace {

thread_local std::string g_error;

int fail(int code, const char* fmt, ...) {
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_error = buf;
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail((int)e, "%s: %s (hipError %d)", what, hipGetErrorString(e), (int)e);
}

#define HIP_TRY(expr)                            \
  do {                                           \
    hipError_t e_ = (expr);                      \
    if (e_ != hipSuccess) return hip_fail(e_, #expr); \
  } while (0)

std::mutex g_mutex;  // guards the cache directory, the plan table and initialisation
// Launches of a plan hold this shared; rl_gemm_plans_clear holds it exclusively while it unloads
// the modules, so a launch never reads a function handle that is being torn down.
std::shared_mutex g_plans_rw;
std::atomic<bool> g_ready{false};  // read without the lock on every entry point
std::atomic<int> g_device{-1};
std::atomic<int> g_lds_limit{0};   // largest LDS allocation of one workgroup, read from the device at rl_init
std::atomic<int> g_compute_units{0};
std::string g_cache_dir;

struct Plan {
  rl_gemm_config cfg;
  hipModule_t module = nullptr;
  hipFunction_t func = nullptr;
  int lds_bytes = 0;
  int lds_limit = 0;  // dynamic LDS the runtime grants this function, read back after load
  int threads = 0;
  int vgprs = -1, agprs = -1, sgprs = -1, spilled = -1, scratch = -1;
  std::string build_log;   // what hiprtc printed for this kernel ("" when the code object came from the disk cache)
};

}  // namespace

struct rl_gemm_plan : Plan {};

namespace {

std::map<std::string, rl_gemm_plan*> g_plans;
// Plans released by rl_gemm_plans_clear: module unloaded, func == nullptr.  The few dozen bytes
// stay allocated so that a handle a caller still holds is refused instead of dereferencing
// freed memory.
std::vector<rl_gemm_plan*> g_released_plans;

// What hiprtc compiles: the work decomposition (which defines the guard that makes the template skip
// its own #include of it) followed by the template.
const std::string& jit_source() {
  static const std::string text = std::string(rl_gemm_sk_decode_begin) + "\n" + rl_gemm_template_begin;
  return text;
}

uint64_t fnv1a(const void* data, size_t n, uint64_t h) {
  const unsigned char* p = (const unsigned char*)data;
  for (size_t i = 0; i < n; ++i) {
    h ^= p[i];
    h *= 1099511628211ull;
  }
  return h;
}

// Same constraints as the static_asserts of the template, reported as text instead of as a
// compiler diagnostic.
int check_config(const rl_gemm_config& c, int* lds_bytes, int* threads) {
  if (c.mi != 32 && c.mi != 16) return fail(RL_ERR_INVALID_ARG, "mi must be 32 or 16, got %d", c.mi);
  if (c.bm <= 0 || c.bn <= 0 || c.bk <= 0 || c.wm <= 0 || c.wn <= 0)
    return fail(RL_ERR_INVALID_ARG, "tile sizes must be positive");
  if (c.bm % c.wm || c.bn % c.wn)
    return fail(RL_ERR_INVALID_ARG, "wave tile %dx%d does not divide block tile %dx%d", c.wm, c.wn, c.bm, c.bn);
  if (c.wm % c.mi || c.wn % c.mi)
    return fail(RL_ERR_INVALID_ARG, "MFMA block %d does not divide wave tile %dx%d", c.mi, c.wm, c.wn);
  const int tn = c.wn / c.mi;
  if ((c.wm / c.mi) * tn > 32)
    return fail(RL_ERR_INVALID_ARG, "wave tile %dx%d is %d MFMA blocks of %d; at most 32 are kept in registers", c.wm, c.wn, (c.wm / c.mi) * tn, c.mi);
  if (c.bn % 4) return fail(RL_ERR_INVALID_ARG, "bn must be a multiple of 4");
  const int ksuper = 4 * (64 / c.mi);
  if (c.bk % ksuper) return fail(RL_ERR_INVALID_ARG, "bk must be a multiple of %d for mi=%d, got %d", ksuper, c.mi, c.bk);
  if (c.pad_a < 0 || c.pad_b < 0 || c.pad_a % 4 || c.pad_b % 4)
    return fail(RL_ERR_INVALID_ARG, "pad_a/pad_b must be non-negative multiples of 4");
  if (c.stages < 1 || c.stages > 5) return fail(RL_ERR_INVALID_ARG, "stages must be 1 to 5, got %d", c.stages);
  if (c.vec != 4 && c.vec != 1) return fail(RL_ERR_INVALID_ARG, "vec must be 4 or 1, got %d", c.vec);
  if (c.edge < 0 || c.edge > 2) return fail(RL_ERR_INVALID_ARG, "edge is 0, 1 or 2, got %d", c.edge);
  if ((c.accum | 1) != 1) return fail(RL_ERR_INVALID_ARG, "accum is 0 or 1");
  if (c.swz < 0 || c.swz > 3) return fail(RL_ERR_INVALID_ARG, "swz is a 2-bit mask");
  if ((c.swz & 2) && c.group <= 0) return fail(RL_ERR_INVALID_ARG, "group must be positive");
  if ((c.direct | 1) != 1) return fail(RL_ERR_INVALID_ARG, "direct is 0 or 1");
  if (c.direct) {
    if (c.stages < 3 || c.pad_a || c.pad_b)
      return fail(RL_ERR_INVALID_ARG, "direct=1 needs stages>=3, pad_a=0, pad_b=0");
    if (c.vec == 1 && (c.stages != 3 || c.edge != 1))
      return fail(RL_ERR_INVALID_ARG, "direct=1 with vec=1 (dword-aligned rows) needs stages=3 and edge=1, got stages=%d edge=%d", c.stages, c.edge);
    if (c.bk & (c.bk - 1)) return fail(RL_ERR_INVALID_ARG, "direct=1 needs bk to be a power of two (XOR swizzle), got %d", c.bk);
    if ((c.bm * c.bk / 4) % 64 || (c.bk * c.bn / 4) % 64)
      return fail(RL_ERR_INVALID_ARG, "direct=1 needs bm*bk and bk*bn to be multiples of 256 (whole waves of 16-byte units)");
  }
  if ((c.trans_b | 1) != 1) return fail(RL_ERR_INVALID_ARG, "trans_b is 0 or 1");
  if (c.streamk < 0 || c.streamk > 8) return fail(RL_ERR_INVALID_ARG, "streamk is 0 (one workgroup per tile) or 1 to 8 workgroups per CU, got %d", c.streamk);
  if (c.streamk && c.stages != 3) return fail(RL_ERR_INVALID_ARG, "streamk needs stages=3 (the pipelined loop with two LDS buffers), got stages=%d", c.stages);
  const int nt = 64 * (c.bm / c.wm) * (c.bn / c.wn);
  if (nt > 1024) return fail(RL_ERR_INVALID_ARG, "%d threads per workgroup exceed 1024", nt);
  const int bufs = c.stages >= 3 ? c.stages - 1 : c.stages;  // LDS buffers: 1, 2, 2, 3, 4
  if (c.stages > 3) {
    if (!c.direct) return fail(RL_ERR_INVALID_ARG, "stages=%d (more than two LDS buffers) needs direct=1", c.stages);
    const int a_units = c.bm * c.bk / 4, b_units = c.bk * c.bn / 4;
    if (a_units % nt || b_units % nt)
      return fail(RL_ERR_INVALID_ARG, "stages=%d needs bm*bk/4 and bk*bn/4 to be multiples of the %d threads", c.stages, nt);
    if ((bufs - 2) * (a_units / nt + b_units / nt) > 63)
      return fail(RL_ERR_INVALID_ARG, "stages=%d keeps %d loads per thread in flight; at most 63", c.stages, (bufs - 2) * (a_units / nt + b_units / nt));
  }
  const long lds = (long)bufs * ((long)c.bm * (c.bk + c.pad_a) + (c.trans_b ? (long)c.bn * (c.bk + c.pad_b) : (long)c.bk * (c.bn + c.pad_b))) * 4;
  if (lds > 160 * 1024) return fail(RL_ERR_INVALID_ARG, "%ld bytes of LDS exceed the 160 KB of a CU", lds);
  if (lds_bytes) *lds_bytes = (int)lds;
  if (threads) *threads = nt;
  return RL_OK;
}

std::vector<std::string> config_options(const rl_gemm_config& c) {
  std::vector<std::string> o;
  auto def = [&](const char* k, int v) { o.push_back(std::string("-D") + k + "=" + std::to_string(v)); };
  def("BM", c.bm); def("BN", c.bn); def("BK", c.bk); def("WM", c.wm); def("WN", c.wn); def("MI", c.mi);
  def("STAGES", c.stages); def("PAD_A", c.pad_a); def("PAD_B", c.pad_b); def("VEC", c.vec);
  def("EDGE", c.edge); def("SWZ", c.swz); def("GROUP", c.group > 0 ? c.group : 1); def("ACCUM", c.accum);
  def("DIRECT", c.direct);
  def("TRANS_B", c.trans_b);
  def("STREAMK", c.streamk);
  return o;
}

std::string config_key(const rl_gemm_config& c) {
  std::string k;
  for (const std::string& s : config_options(c)) k += s + " ";
  return k;
}

const char* const kFixedOptions[] = {"--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
                                     "-Xclang", "-packed-fp32-ops"};

int compile(const char* source, const char* name, const std::vector<std::string>& user_opts,
            std::vector<char>* code, std::string* log) {
  // Fixed part of the command line: the one target this library serves, and no packed-fp32
  // instruction selection.
  std::vector<std::string> all(std::begin(kFixedOptions), std::end(kFixedOptions));
  all.insert(all.end(), user_opts.begin(), user_opts.end());
  std::vector<const char*> argv;
  for (const std::string& s : all) argv.push_back(s.c_str());

  hiprtcProgram prog = nullptr;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, name ? name : "kernel.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail(RL_ERR_COMPILE, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
  r = hiprtcCompileProgram(prog, (int)argv.size(), argv.data());
  size_t log_size = 0;
  if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1 && log) {
    log->resize(log_size);
    hiprtcGetProgramLog(prog, &(*log)[0]);
    while (!log->empty() && log->back() == '\0') log->pop_back();
  }
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    return fail(RL_ERR_COMPILE, "hiprtcCompileProgram: %s\n%s", hiprtcGetErrorString(r), log ? log->c_str() : "");
  }
  size_t n = 0;
  r = hiprtcGetCodeSize(prog, &n);
  if (r == HIPRTC_SUCCESS) {
    code->resize(n);
    r = hiprtcGetCode(prog, code->data());
  }
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS || code->empty())
    return fail(RL_ERR_COMPILE, "hiprtcGetCode: %s", hiprtcGetErrorString(r));
  return RL_OK;
}

std::string cache_path(const rl_gemm_config& c) {
  if (g_cache_dir.empty()) return "";
  // everything that decides the code object: source text, template parameters, the fixed part of the
  // command line, and the compiler -- hiprtc's own version and that of the HIP runtime it ships with
  // (which carries the patch level and changes with every ROCm release)
  int major = 0, minor = 0, runtime = 0;
  hiprtcVersion(&major, &minor);
  (void)hipRuntimeGetVersion(&runtime);
  std::string key = config_key(c) + "|";
  for (const char* o : kFixedOptions) key += std::string(o) + " ";
  key += "|hiprtc " + std::to_string(major) + "." + std::to_string(minor) + " hip " + std::to_string(runtime);
  const std::string& source = jit_source();
  uint64_t h1 = fnv1a(source.data(), source.size(), 14695981039346656037ull);
  h1 = fnv1a(key.data(), key.size(), h1);
  uint64_t h2 = fnv1a(key.data(), key.size(), 0x9e3779b97f4a7c15ull);
  h2 = fnv1a(source.data(), source.size(), h2);
  char name[64];
  snprintf(name, sizeof name, "gemm_%016llx%016llx.hsaco", (unsigned long long)h1, (unsigned long long)h2);
  return g_cache_dir + "/" + name;
}

bool read_file(const std::string& path, std::vector<char>* out) {
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) return false;
  fseek(f, 0, SEEK_END);
  long n = ftell(f);
  fseek(f, 0, SEEK_SET);
  bool ok = n > 0;
  if (ok) {
    out->resize((size_t)n);
    ok = fread(out->data(), 1, (size_t)n, f) == (size_t)n;
  }
  fclose(f);
  return ok;
}

// Write-then-rename so that a concurrent reader never sees half a file.
bool write_file(const std::string& path, const std::vector<char>& data) {
  const std::string tmp = path + ".tmp" + std::to_string((long)getpid());
  FILE* f = fopen(tmp.c_str(), "wb");
  if (!f) return false;
  bool ok = fwrite(data.data(), 1, data.size(), f) == data.size();
  ok = (fclose(f) == 0) && ok;
  if (ok) ok = rename(tmp.c_str(), path.c_str()) == 0;
  if (!ok) unlink(tmp.c_str());
  return ok;
}

// A cache entry is the code object followed by a 16-byte trailer: "RLHC", a format number, and
// the FNV-1a hash of the code object.  An entry that fails this check (cut short, overwritten,
// written by another format) is treated as absent.
constexpr uint32_t kCacheFormat = 1;

void append_trailer(std::vector<char>* data) {
  const uint64_t h = fnv1a(data->data(), data->size(), 14695981039346656037ull);
  char t[16] = {'R', 'L', 'H', 'C'};
  memcpy(t + 4, &kCacheFormat, 4);
  memcpy(t + 8, &h, 8);
  data->insert(data->end(), t, t + 16);
}

bool strip_trailer(std::vector<char>* data) {
  if (data->size() <= 16 + 64) return false;
  const char* t = data->data() + data->size() - 16;
  uint32_t fmt;
  uint64_t h;
  memcpy(&fmt, t + 4, 4);
  memcpy(&h, t + 8, 8);
  if (memcmp(t, "RLHC", 4) != 0 || fmt != kCacheFormat) return false;
  data->resize(data->size() - 16);
  return h == fnv1a(data->data(), data->size(), 14695981039346656037ull) && memcmp(data->data(), "\177ELF", 4) == 0;
}

// Code object for cfg: from the disk cache if present (unless use_cache is false), otherwise
// compiled (and then cached).  *from_cache tells the caller which of the two it got.
int code_for(const rl_gemm_config& c, std::vector<char>* code, float* compile_ms, bool use_cache = true,
             bool* from_cache = nullptr, std::string* build_log = nullptr) {
  if (compile_ms) *compile_ms = 0.0f;
  if (from_cache) *from_cache = false;
  const std::string path = cache_path(c);
  if (use_cache && !path.empty() && read_file(path, code) && strip_trailer(code)) {
    if (from_cache) *from_cache = true;
    return RL_OK;
  }
  code->clear();
  std::string log;
  const auto t0 = std::chrono::steady_clock::now();
  int rc = compile(jit_source().c_str(), "gemm_f32_mfma.hip", config_options(c), code, &log);
  if (build_log) *build_log = log;
  if (rc != RL_OK) return rc;
  if (compile_ms)
    *compile_ms = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
  if (!path.empty()) {
    std::vector<char> entry(*code);
    append_trailer(&entry);
    // A read-only cache directory is not an error for the caller: the kernel is in memory.
    if (!write_file(path, entry)) g_error = "code-object cache not writable: " + path;
  }
  return RL_OK;
}

// Reads an unsigned integer that follows `key` in the msgpack metadata note of a code object.
int metadata_int(const std::vector<char>& code, const char* key) {
  const size_t klen = strlen(key);
  for (size_t i = 0; i + klen + 1 < code.size(); ++i) {
    if (memcmp(&code[i], key, klen) != 0) continue;
    const unsigned char* p = (const unsigned char*)&code[i + klen];
    const size_t left = code.size() - (i + klen);
    if (p[0] <= 0x7f) return p[0];
    if (p[0] == 0xcc && left >= 2) return p[1];
    if (p[0] == 0xcd && left >= 3) return (p[1] << 8) | p[2];
    if (p[0] == 0xce && left >= 5) return (int)(((unsigned)p[1] << 24) | (p[2] << 16) | (p[3] << 8) | p[4]);
  }
  return -1;
}

// The current device is a per-thread setting of the HIP runtime; a thread other than the one that
// called rl_init would otherwise work on device 0.  Every entry point that reaches the runtime
// goes through here; the device is set once per thread.
int ensure_ready() {
  if (!g_ready) return fail(RL_ERR_NO_DEVICE, "rl_init has not been called (or failed)");
  thread_local int t_device = -1;
  if (t_device != g_device) {
    HIP_TRY(hipSetDevice(g_device));
    t_device = g_device;
  }
  return RL_OK;
}

#define READY_OR_RETURN()      \
  do {                         \
    int rc_ = ensure_ready();  \
    if (rc_) return rc_;       \
  } while (0)

// Workgroups that want more than 64 KB of dynamic LDS opt in per function, and the answer is read
// back: *granted receives the dynamic LDS size the runtime will accept for f.  The runtime keys the
// opt-in attribute by host-side kernel stubs; for a function that came from hipModuleGetFunction it
// may answer "invalid device function" (no opt-in exists for module functions).  Only that answer
// is tolerated, and then -- as whenever the function attribute cannot be read -- the grant is the
// device's per-workgroup LDS limit minus the function's static LDS.
int opt_in_lds(hipFunction_t f, int bytes, int* granted) {
  if (bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)f, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipErrorInvalidDeviceFunction) {
      (void)hipGetLastError();  // do not leave a sticky error for the next call
    } else if (e != hipSuccess) {
      return hip_fail(e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
    }
  }
  int static_lds = 0, dynamic_max = 0;
  if (hipFuncGetAttribute(&static_lds, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, f) != hipSuccess) {
    (void)hipGetLastError();
    static_lds = 0;
  }
  if (hipFuncGetAttribute(&dynamic_max, HIP_FUNC_ATTRIBUTE_MAX_DYNAMIC_SHARED_SIZE_BYTES, f) != hipSuccess) {
    (void)hipGetLastError();
    dynamic_max = 0;
  }
  const int device_room = g_lds_limit.load() - static_lds;
  // A function attribute of 0 means "never set": the device limit applies.
  const int limit = dynamic_max > 0 ? (dynamic_max < device_room ? dynamic_max : device_room) : device_room;
  if (granted) *granted = limit;
  if (bytes > limit)
    return fail(RL_ERR_INVALID_ARG, "kernel needs %d bytes of dynamic LDS, the runtime grants %d (device limit %d, static %d, function attribute %d)",
                bytes, limit, g_lds_limit.load(), static_lds, dynamic_max);
  return RL_OK;
}


// ---- stream-K: launch parameters and workspace -------------------------------------------------------

sk_div make_div(unsigned d) {
  // Division of any 32-bit x by the constant d >= 1 (Granlund & Montgomery, the form without a branch):
  // l = ceil(log2 d), mul = floor(2^32 * (2^l - d) / d) + 1, x / d = (t + ((x - t) >> 1)) >> (l - 1) with
  // t = mulhi(x, mul); d = 1 is the same formula with mul = 0 and both shifts 0.
  sk_div out{0u, 0u};
  if (d <= 1) return out;
  unsigned l = 0;
  while ((1ull << l) < d) ++l;
  out.mul = (unsigned)((((1ull << l) - d) << 32) / d + 1);
  out.sh = (1u << 8) | (l - 1);
  return out;
}

// Fills *p for cfg on an M x N x K problem with `compute_units` CUs.  The grid is cfg.streamk
// workgroups per CU, cut down to one K step per workgroup where the problem is smaller than that
// (the decoding relies on no share being empty, unless all are).  Full rounds of the grid are worked
// as whole tiles and only the units of the remaining tiles are shared out.
int sk_make_params(const rl_gemm_config& c, int M, int N, int K, int compute_units, sk_params* p, unsigned* tiles) {
  if (!c.streamk) return fail(RL_ERR_INVALID_ARG, "not a stream-K configuration");
  if (M <= 0 || N <= 0 || K <= 0) return fail(RL_ERR_INVALID_ARG, "stream-K needs M, N, K > 0 (M=%d N=%d K=%d)", M, N, K);
  if (compute_units <= 0) return fail(RL_ERR_INVALID_ARG, "compute_units must be positive");
  const unsigned long nbm = ((unsigned long)M + c.bm - 1) / c.bm, nbn = ((unsigned long)N + c.bn - 1) / c.bn;
  const unsigned long kt = ((unsigned long)K + c.bk - 1) / c.bk;
  const unsigned long units = nbm * nbn * kt;
  if (units >= 0x7fffffffUL || nbm > 0xffffffUL || nbn > 0xffffffUL)
    return fail(RL_ERR_INVALID_ARG, "problem too large for the 32-bit arithmetic of the stream-K split (%lu units)", units);
  unsigned long grid = (unsigned long)compute_units * c.streamk;
  if (grid > units) grid = units;
  const unsigned long n_tiles = nbm * nbn;
  // rounds of whole tiles: all full rounds if the tiles left over are at least a quarter of a round (a
  // tile of theirs is then split four or five ways at most) and no share is empty; else all but one
  // (shares of more than a tile)
  unsigned long rounds = n_tiles / grid;
  if (rounds && (n_tiles % grid) && ((n_tiles % grid) * 4 < grid || (n_tiles % grid) * kt < grid)) --rounds;
  const unsigned long shared = (n_tiles - rounds * grid) * kt;   // units that are shared out
  memset(p, 0, sizeof *p);
  p->grid = (unsigned)grid; p->dp_tiles = (unsigned)(rounds * grid);
  p->q = (unsigned)(shared / grid); p->r = (unsigned)(shared % grid); p->kt = (unsigned)kt;
  p->nbm = (unsigned)nbm; p->nbn = (unsigned)nbn;
  p->group = (c.swz & 2) ? (unsigned)(c.group > 0 ? c.group : 1) : 1u;
  p->rows_last = (unsigned)(nbm % p->group);
  p->d_kt = make_div(p->kt); p->d_q = make_div(p->q); p->d_q1 = make_div(p->q + 1);
  p->d_width = make_div(p->group * p->nbn); p->d_group = make_div(p->group);
  p->d_rows_last = make_div(p->rows_last ? p->rows_last : 1);
  if (tiles) *tiles = (unsigned)(nbm * nbn);
  return RL_OK;
}

// Workspace of one stream-K launch: the arrival counters (one per tile; 256 KiB of them at least, so
// that every launch of up to 65536 tiles keeps them in the same place, then rounded up to 256 bytes),
// then two slots of bm*bn floats per workgroup.  The counter area must be zero when a launch starts
// and is zero again when it ends; the slots may hold anything.  A workspace that is reused for a
// launch with a LARGER counter area has pieces of earlier launches where the new counters go: whoever
// owns the workspace zeroes the counter area again (the library does for its own, below).
size_t sk_counter_bytes(unsigned tiles) {
  const size_t need = ((size_t)tiles * 4 + 255) / 256 * 256;
  return need > RL_STATIC_SCRATCH_COUNTER_BYTES ? need : (size_t)RL_STATIC_SCRATCH_COUNTER_BYTES;
}
size_t sk_workspace_bytes(const rl_gemm_config& c, const sk_params& p, unsigned tiles) {
  return sk_counter_bytes(tiles) + (size_t)2 * p.grid * c.bm * c.bn * 4;
}

// Workspaces the library owns, one per stream (launches on one stream run in order; launches on
// different streams may overlap and must not share counters or slots).  Grown on demand, zeroed
// when allocated (the kernels leave the counters at zero), freed with its stream (rl_stream_destroy);
// the default stream's lives until the process ends.
struct Workspace {
  void* ptr = nullptr;
  size_t bytes = 0;
  size_t counter_bytes = 0;   // the counter area the last launch used (zero from there to the front)
};
std::map<hipStream_t, Workspace> g_workspaces;
std::mutex g_workspaces_mutex;   // (its own lock: launches hold the plan table's shared lock when they get here)

int workspace_for(hipStream_t stream, size_t bytes, size_t counter_bytes, void** out) {
  std::lock_guard<std::mutex> lock(g_workspaces_mutex);
  Workspace& w = g_workspaces[stream];
  if (w.bytes >= bytes && w.counter_bytes != counter_bytes) {
    // the counter area moves its end (only launches of more than 65536 tiles differ): what lies between
    // the two ends held slots of one launch and holds counters of the other.  Zeroed on the launch
    // stream, behind the launches that used the old layout and ahead of the one that uses the new.
    const size_t upto = w.counter_bytes > counter_bytes ? w.counter_bytes : counter_bytes;
    HIP_TRY(hipMemsetAsync(w.ptr, 0, upto, stream));
    w.counter_bytes = counter_bytes;
  }
  if (w.bytes < bytes) {
    if (w.ptr) {
      // the old one may still be in use by a launch queued on this stream
      HIP_TRY(hipStreamSynchronize(stream));
      HIP_TRY(hipFree(w.ptr));
      w = Workspace();
    }
    const size_t want = bytes + bytes / 4;   // head room, so that a slightly larger problem does not reallocate
    HIP_TRY(hipMalloc(&w.ptr, want));
    // zeroed on the launch stream itself: in order with the kernel that follows, also on a stream
    // that does not synchronise with the default stream
    HIP_TRY(hipMemsetAsync(w.ptr, 0, want, stream));
    w.bytes = want;
    w.counter_bytes = counter_bytes;
  }
  *out = w.ptr;
  return RL_OK;
}

enum WorkspaceKind { WS_LIBRARY, WS_CALLER, WS_STATIC };

// Argument checks and launch shared by the plan entry points.  A stream-K plan takes its workspace
// from the library (one per stream) or from the caller.
int launch_plan(const rl_gemm_plan* plan, const float* A, const float* B, float* C, int M, int N, int K,
                int lda, int ldb, int ldc, rl_stream stream, WorkspaceKind kind, void* user_ws, size_t user_ws_bytes) {
  if (!plan) return fail(RL_ERR_INVALID_ARG, "plan is NULL");
  READY_OR_RETURN();
  std::shared_lock<std::shared_mutex> in_flight(g_plans_rw);
  if (!plan->func) return fail(RL_ERR_INVALID_ARG, "plan was released by rl_gemm_plans_clear");
  const rl_gemm_config& c = plan->cfg;
  if (M < 0 || N < 0 || K < 0) return fail(RL_ERR_INVALID_ARG, "negative dimension (M=%d N=%d K=%d)", M, N, K);
  if (M == 0 || N == 0) return RL_OK;
  if (!C || (K > 0 && (!A || !B))) return fail(RL_ERR_INVALID_ARG, "NULL matrix pointer");
  if (lda < K || ldb < (c.trans_b ? K : N) || ldc < N)
    return fail(RL_ERR_INVALID_ARG, "leading dimension too small (lda=%d K=%d, ldb=%d ldc=%d N=%d, trans_b=%d)", lda, K, ldb, ldc, N, c.trans_b);
  if (c.vec == 4) {
    if (K % 4 || N % 4 || lda % 4 || ldb % 4 || ldc % 4)
      return fail(RL_ERR_INVALID_ARG, "vec=4 kernel needs K, N, lda, ldb, ldc to be multiples of 4 (K=%d N=%d lda=%d ldb=%d ldc=%d)", K, N, lda, ldb, ldc);
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15)
      return fail(RL_ERR_INVALID_ARG, "vec=4 kernel needs 16-byte aligned A, B and C");
  } else if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 3) {
    return fail(RL_ERR_INVALID_ARG, "A, B and C must be 4-byte aligned");
  }
  if (!c.edge && (M % c.bm || N % c.bn || K % c.bk))
    return fail(RL_ERR_INVALID_ARG, "edge=0 kernel needs bm|M, bn|N, bk|K (tile %dx%dx%d, problem %dx%dx%d)", c.bm, c.bn, c.bk, M, N, K);
  if (c.edge == 2 && K % c.bk)
    return fail(RL_ERR_INVALID_ARG, "edge=2 kernel needs bk|K (bk=%d, K=%d)", c.bk, K);
  // In-tile byte offsets are 32-bit inside the kernel; 0x80000000 is reserved as "out of range".
  const long lim = 0x7fffffffL;
  if ((long)c.bm * lda * 4 + (long)c.bk * 4 > lim || (c.trans_b ? (long)c.bn * ldb * 4 + (long)c.bk * 4 : (long)c.bk * ldb * 4 + (long)c.bn * 4) > lim ||
      (long)c.bm * ldc * 4 + (long)c.bn * 4 > lim)
    return fail(RL_ERR_INVALID_ARG, "leading dimension too large for 32-bit in-tile offsets");
  const long nbm = ((long)M + c.bm - 1) / c.bm, nbn = ((long)N + c.bn - 1) / c.bn;
  if (nbn > 0x7fffffffL || nbm > 65535 || nbm * nbn > lim)
    return fail(RL_ERR_INVALID_ARG, "tile grid %ldx%ld too large", nbn, nbm);

  if (!c.streamk) {
    void* args[] = {(void*)&A, (void*)&B, (void*)&C, &M, &N, &K, &lda, &ldb, &ldc};
    HIP_TRY(hipModuleLaunchKernel(plan->func, (unsigned)nbn, (unsigned)nbm, 1, (unsigned)plan->threads, 1, 1,
                                  (unsigned)plan->lds_bytes, (hipStream_t)stream, args, nullptr));
    return RL_OK;
  }

  if (K == 0) {
    // no K step to hand out: C = 0 (or C unchanged when accumulating), without the kernel
    if (!c.accum) HIP_TRY(rl_scratch_zero_c(C, ldc, M, N, (hipStream_t)stream));
    return RL_OK;
  }
  sk_params sp;
  unsigned tiles = 0;
  int rc = sk_make_params(c, M, N, K, g_compute_units.load(), &sp, &tiles);
  if (rc) return rc;
  const size_t need = sk_workspace_bytes(c, sp, tiles);
  void* ws = nullptr;
  // the counters sit at the front of a workspace; the static array keeps a fixed room for them
  size_t counter_room = sk_counter_bytes(tiles);
  if (kind == WS_STATIC) {
    ws = rl_scratch_address(g_device.load());
    if (!ws) return fail(RL_ERR_NO_DEVICE, "the static scratch array was not set up (rl_init)");
    counter_room = RL_STATIC_SCRATCH_COUNTER_BYTES;
    const size_t slots = need - sk_counter_bytes(tiles);
    if (sk_counter_bytes(tiles) > counter_room || slots > RL_STATIC_SCRATCH_BYTES - counter_room)
      return fail(RL_ERR_INVALID_ARG, "rl_gemm_plan_launch_static: this launch needs %zu bytes of counters and %zu bytes of slots; the static scratch array holds %u and %u (use rl_gemm_plan_launch or rl_gemm_plan_launch_ws)",
                  sk_counter_bytes(tiles), slots, RL_STATIC_SCRATCH_COUNTER_BYTES, RL_STATIC_SCRATCH_BYTES - RL_STATIC_SCRATCH_COUNTER_BYTES);
  } else if (kind == WS_CALLER) {
    if (!user_ws || user_ws_bytes < need)
      return fail(RL_ERR_INVALID_ARG, "stream-K launch needs a workspace of %zu bytes (rl_gemm_plan_workspace_bytes), got %zu", need, user_ws ? user_ws_bytes : (size_t)0);
    if ((uintptr_t)user_ws & 255) return fail(RL_ERR_INVALID_ARG, "workspace must be 256-byte aligned");
    ws = user_ws;
  } else {
    rc = workspace_for((hipStream_t)stream, need, counter_room, &ws);
    if (rc) return rc;
  }
  unsigned* arrivals = (unsigned*)ws;
  float* slots = (float*)((char*)ws + counter_room);
  void* args[] = {(void*)&A, (void*)&B, (void*)&C, &M, &N, &K, &lda, &ldb, &ldc, &slots, &arrivals, &sp};
  HIP_TRY(hipModuleLaunchKernel(plan->func, sp.grid, 1, 1, (unsigned)plan->threads, 1, 1,
                                (unsigned)plan->lds_bytes, (hipStream_t)stream, args, nullptr));
  return RL_OK;
}

}  // namespace

extern "C" {

int rl_init(int device) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_ready && g_device == device) return RL_OK;
  if (g_ready)  // loaded modules, streams and allocations belong to the first device
    return fail(RL_ERR_INVALID_ARG, "already initialised on device %d; one device per process", g_device.load());
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0)
    return fail(RL_ERR_NO_DEVICE, "no HIP device visible (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
  if (device < 0 || device >= count)
    return fail(RL_ERR_INVALID_ARG, "device %d out of range (0..%d)", device, count - 1);
  HIP_TRY(hipSetDevice(device));
  HIP_TRY(hipFree(nullptr));  // forces context creation
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(RL_ERR_NO_DEVICE, "device %d is %s; this library is built for gfx950 (MI355X) only", device, prop.gcnArchName);
  int lds_limit = (int)prop.sharedMemPerBlockOptin > 0 ? (int)prop.sharedMemPerBlockOptin : (int)prop.sharedMemPerBlock;
  int attr = 0;
  if (hipDeviceGetAttribute(&attr, hipDeviceAttributeMaxSharedMemoryPerBlock, device) == hipSuccess && attr > lds_limit)
    lds_limit = attr;
  // where this device keeps the library's static scratch array (rl_gemm_plan_launch_static)
  HIP_TRY(rl_scratch_setup(device));
  g_lds_limit = lds_limit;
  g_compute_units = prop.multiProcessorCount;
  g_device = device;
  g_ready = true;
  return RL_OK;
}

int rl_device_info(rl_device_props* out) {
  if (!out) return fail(RL_ERR_INVALID_ARG, "out is NULL");
  int rc = ensure_ready();
  if (rc) return rc;
  hipDeviceProp_t p;
  HIP_TRY(hipGetDeviceProperties(&p, g_device));
  memset(out, 0, sizeof *out);
  snprintf(out->name, sizeof out->name, "%.127s", p.name);
  snprintf(out->arch, sizeof out->arch, "%.63s", p.gcnArchName);
  out->compute_units = p.multiProcessorCount;
  out->wavefront_size = p.warpSize;
  out->lds_bytes_per_block = g_lds_limit.load();
  out->regs_per_block = p.regsPerBlock;
  out->l2_bytes = p.l2CacheSize;
  out->clock_khz = p.clockRate;
  out->mem_clock_khz = p.memoryClockRate;
  out->mem_bus_bits = p.memoryBusWidth;
  out->total_mem_bytes = p.totalGlobalMem;
  return RL_OK;
}

const char* rl_last_error(void) { return g_error.c_str(); }

int rl_compile(const char* source, const char* name, const char* const* options, int n_options,
               void** code, size_t* code_size, char** log) {
  if (log) *log = nullptr;
  if (!source || !code || !code_size || n_options < 0 || (n_options > 0 && !options))
    return fail(RL_ERR_INVALID_ARG, "rl_compile: NULL argument");
  *code = nullptr;
  *code_size = 0;
  std::vector<std::string> opts;
  for (int i = 0; i < n_options; ++i) opts.push_back(options[i] ? options[i] : "");
  std::vector<char> obj;
  std::string text;
  int rc = compile(source, name, opts, &obj, &text);
  if (log) {
    *log = (char*)malloc(text.size() + 1);
    if (*log) memcpy(*log, text.c_str(), text.size() + 1);
  }
  if (rc != RL_OK) return rc;
  *code = malloc(obj.size());
  if (!*code) return fail(RL_ERR_IO, "out of host memory");
  memcpy(*code, obj.data(), obj.size());
  *code_size = obj.size();
  return RL_OK;
}

void rl_free_host(void* p) { free(p); }

int rl_module_load(const void* code, rl_module* out) {
  if (!code || !out) return fail(RL_ERR_INVALID_ARG, "rl_module_load: NULL argument");
  int rc = ensure_ready();
  if (rc) return rc;
  hipModule_t m = nullptr;
  HIP_TRY(hipModuleLoadData(&m, code));
  *out = m;
  return RL_OK;
}

int rl_module_get_function(rl_module m, const char* name, rl_function* out) {
  if (!m || !name || !out) return fail(RL_ERR_INVALID_ARG, "rl_module_get_function: NULL argument");
  READY_OR_RETURN();
  hipFunction_t f = nullptr;
  HIP_TRY(hipModuleGetFunction(&f, (hipModule_t)m, name));
  *out = f;
  return RL_OK;
}

int rl_module_unload(rl_module m) {
  if (!m) return RL_OK;
  READY_OR_RETURN();
  // kernels of this module may still be queued (a host wrapper's destructor can get here right
  // after its last launch): let them finish before their code goes away
  HIP_TRY(hipDeviceSynchronize());
  HIP_TRY(hipModuleUnload((hipModule_t)m));
  return RL_OK;
}

int rl_func_set_max_dynamic_lds(rl_function f, int bytes) {
  if (!f || bytes < 0) return fail(RL_ERR_INVALID_ARG, "rl_func_set_max_dynamic_lds: bad argument");
  if (bytes > 160 * 1024) return fail(RL_ERR_INVALID_ARG, "%d bytes of LDS exceed the 160 KB of a CU", bytes);
  READY_OR_RETURN();
  return opt_in_lds((hipFunction_t)f, bytes, nullptr);
}

int rl_launch(rl_function f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
              unsigned bz, unsigned lds_bytes, rl_stream stream, void** args, int n_args) {
  if (!f || (n_args > 0 && !args)) return fail(RL_ERR_INVALID_ARG, "rl_launch: NULL argument");
  if (!gx || !gy || !gz || !bx || !by || !bz) return fail(RL_ERR_INVALID_ARG, "rl_launch: empty grid or block");
  if ((unsigned long)bx * by * bz > 1024) return fail(RL_ERR_INVALID_ARG, "rl_launch: more than 1024 threads per block");
  for (int i = 0; i < n_args; ++i)
    if (!args[i]) return fail(RL_ERR_INVALID_ARG, "rl_launch: args[%d] is NULL", i);
  if ((long)lds_bytes > g_lds_limit.load() && g_ready)
    return fail(RL_ERR_INVALID_ARG, "rl_launch: %u bytes of dynamic LDS exceed the device's %d per workgroup", lds_bytes, g_lds_limit.load());
  READY_OR_RETURN();
  HIP_TRY(hipModuleLaunchKernel((hipFunction_t)f, gx, gy, gz, bx, by, bz, lds_bytes, (hipStream_t)stream, args, nullptr));
  return RL_OK;
}

int rl_malloc(void** dptr, size_t bytes) {
  if (!dptr) return fail(RL_ERR_INVALID_ARG, "rl_malloc: NULL argument");
  int rc = ensure_ready();
  if (rc) return rc;
  *dptr = nullptr;
  if (bytes == 0) return RL_OK;
  HIP_TRY(hipMalloc(dptr, bytes));
  return RL_OK;
}

int rl_free(void* dptr) {
  if (!dptr) return RL_OK;
  READY_OR_RETURN();
  HIP_TRY(hipFree(dptr));
  return RL_OK;
}

int rl_memcpy_h2d(void* dst, const void* src, size_t bytes) {
  if (bytes == 0) return RL_OK;
  if (!dst || !src) return fail(RL_ERR_INVALID_ARG, "rl_memcpy_h2d: NULL argument");
  READY_OR_RETURN();
  HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return RL_OK;
}

int rl_memcpy_d2h(void* dst, const void* src, size_t bytes) {
  if (bytes == 0) return RL_OK;
  if (!dst || !src) return fail(RL_ERR_INVALID_ARG, "rl_memcpy_d2h: NULL argument");
  READY_OR_RETURN();
  HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return RL_OK;
}

int rl_memset(void* dptr, int byte_value, size_t bytes) {
  if (bytes == 0) return RL_OK;
  if (!dptr) return fail(RL_ERR_INVALID_ARG, "rl_memset: NULL argument");
  READY_OR_RETURN();
  HIP_TRY(hipMemset(dptr, byte_value, bytes));
  return RL_OK;
}

int rl_stream_create(rl_stream* out) {
  if (!out) return fail(RL_ERR_INVALID_ARG, "rl_stream_create: NULL argument");
  int rc = ensure_ready();
  if (rc) return rc;
  hipStream_t s = nullptr;
  HIP_TRY(hipStreamCreate(&s));  // default priority on purpose
  *out = s;
  return RL_OK;
}

int rl_stream_destroy(rl_stream s) {
  if (!s) return RL_OK;
  READY_OR_RETURN();
  {
    // the stream's stream-K workspace goes with it (a later stream may get the same handle value, and a
    // process that makes and drops streams must not keep 64 MiB for each)
    std::lock_guard<std::mutex> lock(g_workspaces_mutex);
    auto it = g_workspaces.find((hipStream_t)s);
    if (it != g_workspaces.end()) {
      if (it->second.ptr) {
        HIP_TRY(hipStreamSynchronize((hipStream_t)s));
        HIP_TRY(hipFree(it->second.ptr));
      }
      g_workspaces.erase(it);
    }
  }
  HIP_TRY(hipStreamDestroy((hipStream_t)s));
  return RL_OK;
}

int rl_event_create(rl_event* out) {
  if (!out) return fail(RL_ERR_INVALID_ARG, "rl_event_create: NULL argument");
  int rc = ensure_ready();
  if (rc) return rc;
  hipEvent_t e = nullptr;
  HIP_TRY(hipEventCreate(&e));
  *out = e;
  return RL_OK;
}

int rl_event_record(rl_event e, rl_stream s) {
  if (!e) return fail(RL_ERR_INVALID_ARG, "rl_event_record: NULL event");
  READY_OR_RETURN();
  HIP_TRY(hipEventRecord((hipEvent_t)e, (hipStream_t)s));
  return RL_OK;
}

int rl_event_sync(rl_event e) {
  if (!e) return fail(RL_ERR_INVALID_ARG, "rl_event_sync: NULL event");
  READY_OR_RETURN();
  HIP_TRY(hipEventSynchronize((hipEvent_t)e));
  return RL_OK;
}

int rl_event_elapsed_ms(rl_event start, rl_event stop, float* ms) {
  if (!start || !stop || !ms) return fail(RL_ERR_INVALID_ARG, "rl_event_elapsed_ms: NULL argument");
  READY_OR_RETURN();
  HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
  return RL_OK;
}

int rl_event_destroy(rl_event e) {
  if (!e) return RL_OK;
  READY_OR_RETURN();
  HIP_TRY(hipEventDestroy((hipEvent_t)e));
  return RL_OK;
}

int rl_sync(void) {
  int rc = ensure_ready();
  if (rc) return rc;
  HIP_TRY(hipDeviceSynchronize());
  return RL_OK;
}

const char* rl_gemm_template_source(void) { return jit_source().c_str(); }

int rl_gemm_config_check(const rl_gemm_config* cfg, int* lds_bytes, int* threads) {
  if (!cfg) return fail(RL_ERR_INVALID_ARG, "cfg is NULL");
  return check_config(*cfg, lds_bytes, threads);
}

int rl_set_cache_dir(const char* path) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!path || !*path) {
    g_cache_dir.clear();
    return RL_OK;
  }
  struct stat st;
  if (stat(path, &st) != 0) {
    if (mkdir(path, 0777) != 0) return fail(RL_ERR_IO, "cannot create cache directory %s", path);
  } else if (!S_ISDIR(st.st_mode)) {
    return fail(RL_ERR_IO, "%s is not a directory", path);
  }
  g_cache_dir = path;
  return RL_OK;
}

int rl_gemm_precompile(const rl_gemm_config* cfg, size_t* code_size) {
  if (!cfg) return fail(RL_ERR_INVALID_ARG, "cfg is NULL");
  int rc = check_config(*cfg, nullptr, nullptr);
  if (rc) return rc;
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_cache_dir.empty()) return fail(RL_ERR_IO, "rl_gemm_precompile needs a cache directory (rl_set_cache_dir)");
  std::vector<char> code;
  rc = code_for(*cfg, &code, nullptr);
  if (rc) return rc;
  std::vector<char> check;
  if (!read_file(cache_path(*cfg), &check) || !strip_trailer(&check))
    return fail(RL_ERR_IO, "could not store %s", cache_path(*cfg).c_str());
  if (code_size) *code_size = code.size();
  return RL_OK;
}

int rl_gemm_plan_create(const rl_gemm_config* cfg, rl_gemm_plan** out, float* compile_ms) {
  if (compile_ms) *compile_ms = 0.0f;
  if (!cfg || !out) return fail(RL_ERR_INVALID_ARG, "rl_gemm_plan_create: NULL argument");
  *out = nullptr;
  int lds = 0, threads = 0;
  int rc = check_config(*cfg, &lds, &threads);
  if (rc) return rc;
  rc = ensure_ready();
  if (rc) return rc;

  std::lock_guard<std::mutex> lock(g_mutex);
  const std::string key = config_key(*cfg);
  auto it = g_plans.find(key);
  if (it != g_plans.end()) {
    *out = it->second;
    return RL_OK;
  }
  std::vector<char> code;
  bool from_cache = false;
  std::string build_log;
  rc = code_for(*cfg, &code, compile_ms, true, &from_cache, &build_log);
  if (rc) return rc;

  rl_gemm_plan* p = new rl_gemm_plan();
  p->build_log = build_log;
  p->cfg = *cfg;
  p->lds_bytes = lds;
  p->threads = threads;
  hipError_t e = hipSuccess;
  for (int attempt = 0; attempt < 2; ++attempt) {
    e = hipModuleLoadData(&p->module, code.data());
    if (e == hipSuccess) e = hipModuleGetFunction(&p->func, p->module, "gemm_kernel");
    if (e == hipSuccess || !from_cache) break;
    // A cached file that does not load (damaged, or written for another driver) is replaced once.
    (void)hipGetLastError();
    if (p->module) (void)hipModuleUnload(p->module);
    p->module = nullptr;
    p->func = nullptr;
    from_cache = false;
    rc = code_for(*cfg, &code, compile_ms, false, nullptr, &p->build_log);
    if (rc) {
      delete p;
      return rc;
    }
  }
  if (e != hipSuccess) {
    if (p->module) (void)hipModuleUnload(p->module);
    delete p;
    return hip_fail(e, "loading the compiled GEMM kernel");
  }
  // opt in to the plan's LDS size and read back what the runtime grants: a refusal is reported
  // here, with text, and not by the first launch
  rc = opt_in_lds(p->func, lds, &p->lds_limit);
  if (rc) {
    (void)hipModuleUnload(p->module);
    delete p;
    return rc;
  }
  p->vgprs = metadata_int(code, ".vgpr_count");
  p->agprs = metadata_int(code, ".agpr_count");
  p->sgprs = metadata_int(code, ".sgpr_count");
  const int vs = metadata_int(code, ".vgpr_spill_count"), ss = metadata_int(code, ".sgpr_spill_count");
  p->spilled = (vs < 0 || ss < 0) ? -1 : vs + ss;
  p->scratch = metadata_int(code, ".private_segment_fixed_size");
  g_plans[key] = p;
  *out = p;
  return RL_OK;
}

int rl_gemm_plan_function(const rl_gemm_plan* plan, rl_function* out) {
  if (!plan || !out) return fail(RL_ERR_INVALID_ARG, "rl_gemm_plan_function: NULL argument");
  std::shared_lock<std::shared_mutex> in_flight(g_plans_rw);
  if (!plan->func) return fail(RL_ERR_INVALID_ARG, "plan was released by rl_gemm_plans_clear");
  *out = plan->func;
  return RL_OK;
}

int rl_gemm_plan_lds_bytes(const rl_gemm_plan* plan) { return plan ? plan->lds_bytes : 0; }
int rl_gemm_plan_lds_limit(const rl_gemm_plan* plan) { return plan ? plan->lds_limit : 0; }
int rl_gemm_plan_threads(const rl_gemm_plan* plan) { return plan ? plan->threads : 0; }

int rl_gemm_plan_resources(const rl_gemm_plan* plan, int* vgprs, int* agprs, int* sgprs,
                           int* spilled, int* scratch_bytes) {
  if (!plan) return fail(RL_ERR_INVALID_ARG, "plan is NULL");
  if (vgprs) *vgprs = plan->vgprs;
  if (agprs) *agprs = plan->agprs;
  if (sgprs) *sgprs = plan->sgprs;
  if (spilled) *spilled = plan->spilled;
  if (scratch_bytes) *scratch_bytes = plan->scratch;
  return RL_OK;
}

const char* rl_gemm_plan_build_log(const rl_gemm_plan* plan) { return plan ? plan->build_log.c_str() : ""; }

int rl_gemm_plans_clear(void) {
  READY_OR_RETURN();
  std::lock_guard<std::mutex> lock(g_mutex);
  std::unique_lock<std::shared_mutex> no_launches(g_plans_rw);
  // launches enqueued earlier may still be running the code that is about to be unloaded
  HIP_TRY(hipDeviceSynchronize());
  int rc = RL_OK;
  for (auto& kv : g_plans) {
    if (kv.second->module) {
      hipError_t e = hipModuleUnload(kv.second->module);
      if (e != hipSuccess) rc = hip_fail(e, "hipModuleUnload");
    }
    kv.second->module = nullptr;
    kv.second->func = nullptr;
    g_released_plans.push_back(kv.second);
  }
  g_plans.clear();
  return rc;
}

int rl_gemm_plan_launch(const rl_gemm_plan* plan, const float* A, const float* B, float* C,
                        int M, int N, int K, int lda, int ldb, int ldc, rl_stream stream) {
  return launch_plan(plan, A, B, C, M, N, K, lda, ldb, ldc, stream, WS_LIBRARY, nullptr, 0);
}

int rl_gemm_plan_launch_ws(const rl_gemm_plan* plan, const float* A, const float* B, float* C,
                           int M, int N, int K, int lda, int ldb, int ldc, void* workspace,
                           size_t workspace_bytes, rl_stream stream) {
  return launch_plan(plan, A, B, C, M, N, K, lda, ldb, ldc, stream, WS_CALLER, workspace, workspace_bytes);
}

int rl_gemm_plan_launch_static(const rl_gemm_plan* plan, const float* A, const float* B, float* C,
                               int M, int N, int K, int lda, int ldb, int ldc, rl_stream stream) {
  return launch_plan(plan, A, B, C, M, N, K, lda, ldb, ldc, stream, WS_STATIC, nullptr, 0);
}

int rl_gemm_plan_workspace_bytes(const rl_gemm_plan* plan, int M, int N, int K, size_t* bytes, size_t* counter_bytes) {
  if (!plan || !bytes) return fail(RL_ERR_INVALID_ARG, "rl_gemm_plan_workspace_bytes: NULL argument");
  *bytes = 0;
  if (counter_bytes) *counter_bytes = 0;
  if (!plan->cfg.streamk || M <= 0 || N <= 0 || K <= 0) return RL_OK;
  READY_OR_RETURN();
  sk_params sp;
  unsigned tiles = 0;
  int rc = sk_make_params(plan->cfg, M, N, K, g_compute_units.load(), &sp, &tiles);
  if (rc) return rc;
  *bytes = sk_workspace_bytes(plan->cfg, sp, tiles);
  if (counter_bytes) *counter_bytes = sk_counter_bytes(tiles);
  return RL_OK;
}

int rl_gemm_streamk_schedule(const rl_gemm_config* cfg, int M, int N, int K, int compute_units,
                             rl_streamk_schedule* out) {
  if (!cfg || !out) return fail(RL_ERR_INVALID_ARG, "rl_gemm_streamk_schedule: NULL argument");
  int rc = check_config(*cfg, nullptr, nullptr);
  if (rc) return rc;
  sk_params sp;
  unsigned tiles = 0;
  rc = sk_make_params(*cfg, M, N, K, compute_units, &sp, &tiles);
  if (rc) return rc;
  memset(out, 0, sizeof *out);
  out->grid = (int)sp.grid;
  out->k_steps = (int)sp.kt;
  out->tiles = (int)tiles;
  out->tile_rows = (int)sp.nbm;
  out->tile_cols = (int)sp.nbn;
  out->units = (long)tiles * sp.kt;
  out->whole_tiles = (int)sp.dp_tiles;
  out->workspace_bytes = sk_workspace_bytes(*cfg, sp, tiles);
  out->counter_bytes = sk_counter_bytes(tiles);
  return RL_OK;
}

int rl_gemm_streamk_segments(const rl_gemm_config* cfg, int M, int N, int K, int compute_units,
                             int workgroup, rl_streamk_segment* out, int capacity, int* count) {
  if (!cfg || !count || (capacity > 0 && !out)) return fail(RL_ERR_INVALID_ARG, "rl_gemm_streamk_segments: NULL argument");
  int rc = check_config(*cfg, nullptr, nullptr);
  if (rc) return rc;
  sk_params sp;
  rc = sk_make_params(*cfg, M, N, K, compute_units, &sp, nullptr);
  if (rc) return rc;
  if (workgroup < 0 || (unsigned)workgroup >= sp.grid)
    return fail(RL_ERR_INVALID_ARG, "workgroup %d out of range (grid %u)", workgroup, sp.grid);
  // exactly what a workgroup of the kernel does with its (logical) index
  unsigned unit = sk_first_unit(sp, (unsigned)workgroup);
  const unsigned end = sk_first_unit(sp, (unsigned)workgroup + 1);
  unsigned whole = (unsigned)workgroup;
  int n = 0;
  while (unit < end || whole < sp.dp_tiles) {
    sk_segment seg;
    if (unit < end) {
      seg = sk_segment_at(sp, unit, end);
      unit += seg.ke - seg.kb;
    } else {
      seg = sk_whole_tile(sp, whole);
      whole += sp.grid;
    }
    if (n < capacity) {
      rl_streamk_segment& o = out[n];
      o.tile = (int)seg.tile; o.tile_m = (int)seg.tile_m; o.tile_n = (int)seg.tile_n;
      o.k_begin = (int)seg.kb; o.k_end = (int)seg.ke;
      o.pieces = 1; o.first_workgroup = workgroup; o.slot = -1;
      if (seg.kb != 0 || seg.ke != sp.kt) {
        const unsigned first_wg = sk_owner(sp, sk_tile_unit(sp, seg.tile));
        o.first_workgroup = (int)first_wg;
        o.pieces = (int)(sk_owner(sp, sk_tile_unit(sp, seg.tile) + sp.kt - 1) - first_wg + 1);
        o.slot = 2 * workgroup + (seg.kb == 0 ? 1 : 0);
      }
    }
    ++n;
  }
  *count = n;
  return RL_OK;
}

int rl_gemm_f32(const rl_gemm_config* cfg, const float* A, const float* B, float* C, int M,
                int N, int K, int lda, int ldb, int ldc, rl_stream stream) {
  rl_gemm_plan* plan = nullptr;
  int rc = rl_gemm_plan_create(cfg, &plan, nullptr);
  if (rc) return rc;
  return rl_gemm_plan_launch(plan, A, B, C, M, N, K, lda, ldb, ldc, stream);
}

}  // extern "C"
