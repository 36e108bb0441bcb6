// frnn_rt: C-ABI runtime for generated gfx950 kernels (see include/frnn_rt.h).
//
// Host-only C++; the HIP runtime is resolved at run time from the process image
// (dlsym(RTLD_DEFAULT)) so that the copy PyTorch already loaded is the one used, and is
// dlopen'ed by soname only when the process has none.
#include "frnn_rt.h"
#include "frnn_internal.h"

#include <dlfcn.h>
#include <errno.h>
#include <fcntl.h>
#include <spawn.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/file.h>
#include <sys/stat.h>
#include <sys/wait.h>
#include <unistd.h>

#include <mutex>
#include <string>
#include <vector>

extern char** environ;

namespace {

thread_local std::string g_err;

int fail(int code, const char* fmt, ...) {
  char buf[4096];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_err = buf;
  return code;
}

void set_error(const char* msg) { g_err = msg; }

// ---------------------------------------------------------------- HIP entry points
typedef int hipError_t;
struct HipApi {
  hipError_t (*ModuleLoadData)(void**, const void*) = nullptr;
  hipError_t (*ModuleUnload)(void*) = nullptr;
  hipError_t (*ModuleGetFunction)(void**, void*, const char*) = nullptr;
  hipError_t (*ModuleLaunchKernel)(void*, unsigned, unsigned, unsigned, unsigned, unsigned, unsigned,
                                   unsigned, void*, void**, void**) = nullptr;
  const char* (*GetErrorString)(hipError_t) = nullptr;
  hipError_t (*GetDevice)(int*) = nullptr;
  hipError_t (*DeviceGetAttribute)(int*, int, int) = nullptr;
  hipError_t (*GetLastError)() = nullptr;
  bool ok = false;
  std::string why;
};

HipApi& hip() {
  static HipApi api;
  static std::once_flag once;
  std::call_once(once, [] {
    void* h = RTLD_DEFAULT;
    if (!dlsym(RTLD_DEFAULT, "hipModuleLoadData")) {
      h = dlopen("libamdhip64.so", RTLD_NOW | RTLD_GLOBAL);
      if (!h) h = dlopen("libamdhip64.so.7", RTLD_NOW | RTLD_GLOBAL);
      if (!h) h = dlopen("/opt/rocm/lib/libamdhip64.so", RTLD_NOW | RTLD_GLOBAL);
      if (!h) {
        api.why = "no HIP runtime in the process and libamdhip64.so could not be loaded";
        return;
      }
    }
#define FRNN_SYM(field, name)                                              \
  *(void**)(&api.field) = dlsym(h, name);                                  \
  if (!api.field) { api.why = std::string("missing HIP symbol ") + name; return; }
    FRNN_SYM(ModuleLoadData, "hipModuleLoadData")
    FRNN_SYM(ModuleUnload, "hipModuleUnload")
    FRNN_SYM(ModuleGetFunction, "hipModuleGetFunction")
    FRNN_SYM(ModuleLaunchKernel, "hipModuleLaunchKernel")
    FRNN_SYM(GetErrorString, "hipGetErrorString")
    FRNN_SYM(GetDevice, "hipGetDevice")
    FRNN_SYM(DeviceGetAttribute, "hipDeviceGetAttribute")
    FRNN_SYM(GetLastError, "hipGetLastError")
#undef FRNN_SYM
    api.ok = true;
  });
  return api;
}

int hip_fail(const char* what, hipError_t e) {
  const char* s = hip().GetErrorString ? hip().GetErrorString(e) : "?";
  return fail(FRNN_ERR_HIP, "%s failed: %s (%d)", what, s, (int)e);
}

// ---------------------------------------------------------------- small file helpers
bool file_exists(const std::string& p) {
  struct stat st;
  return stat(p.c_str(), &st) == 0 && S_ISREG(st.st_mode) && st.st_size > 0;
}

int mkdirs(const std::string& dir) {
  std::string cur;
  for (size_t i = 0; i <= dir.size(); i++) {
    if (i == dir.size() || dir[i] == '/') {
      if (!cur.empty() && mkdir(cur.c_str(), 0777) != 0 && errno != EEXIST) return -1;
    }
    if (i < dir.size()) cur.push_back(dir[i]);
  }
  return 0;
}

int write_file(const std::string& path, const char* data, size_t len) {
  FILE* f = fopen(path.c_str(), "wb");
  if (!f) return -1;
  size_t w = fwrite(data, 1, len, f);
  int rc = fclose(f);
  return (w == len && rc == 0) ? 0 : -1;
}

std::string read_tail(const std::string& path, size_t maxb) {
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) return "";
  fseek(f, 0, SEEK_END);
  long n = ftell(f);
  long off = n > (long)maxb ? n - (long)maxb : 0;
  fseek(f, off, SEEK_SET);
  std::string s((size_t)(n - off), '\0');
  size_t r = fread(&s[0], 1, s.size(), f);
  s.resize(r);
  fclose(f);
  return s;
}

std::string find_hipcc() {
  if (const char* e = getenv("FRNN_HIPCC")) return e;
  if (const char* r = getenv("ROCM_PATH")) {
    std::string p = std::string(r) + "/bin/hipcc";
    if (access(p.c_str(), X_OK) == 0) return p;
  }
  if (access("/opt/rocm/bin/hipcc", X_OK) == 0) return "/opt/rocm/bin/hipcc";
  return "hipcc";
}

std::vector<std::string> split_ws(const char* s) {
  std::vector<std::string> out;
  if (!s) return out;
  std::string cur;
  for (const char* p = s;; p++) {
    if (*p == 0 || *p == ' ' || *p == '\t' || *p == '\n') {
      if (!cur.empty()) out.push_back(cur);
      cur.clear();
      if (*p == 0) break;
    } else {
      cur.push_back(*p);
    }
  }
  return out;
}

}  // namespace

int frnn_detail_fail(int code, const char* fmt, ...) {
  char buf[4096];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  set_error(buf);
  return code;
}

struct frnn_module_s {
  void* mod;
  std::vector<char> image;   // the code object bytes; kept for the lifetime of the module
  std::vector<frnn_kernel_s*> kernels;   // handles given out by frnn_get_kernel; freed with the module
  std::mutex mu;                         // guards `kernels`
};

namespace {

// ---------------------------------------------------------------- code object metadata
// The AMDGPU metadata note of a code object is a MessagePack map
//   { "amdhsa.kernels": [ { ".name": <str>, ".kernarg_segment_size": <uint>, ... }, ... ], ... }.
// Only what is needed to read that one number is implemented.
struct MsgPack {
  const uint8_t* p;
  const uint8_t* e;
  bool ok = true;

  uint64_t be(int n) {
    if (e - p < n) { ok = false; return 0; }
    uint64_t v = 0;
    for (int i = 0; i < n; i++) v = (v << 8) | *p++;
    return v;
  }
  bool str(const char** s, size_t* n) {         // consumes a string; false (nothing consumed) for another type
    if (p >= e) return ok = false;
    const uint8_t t = *p;
    const uint8_t* save = p;
    size_t len;
    if (t >= 0xa0 && t <= 0xbf) { len = t & 0x1f; p++; }
    else if (t == 0xd9 || t == 0xda || t == 0xdb) { p++; len = (size_t)be(t == 0xd9 ? 1 : t == 0xda ? 2 : 4); }
    else return false;
    if (!ok || (size_t)(e - p) < len) { p = save; return ok = false; }
    *s = (const char*)p; *n = len; p += len;
    return true;
  }
  bool uint_(uint64_t* v) {
    if (p >= e) return ok = false;
    uint8_t t = *p;
    if (t <= 0x7f) { *v = t; p++; return true; }
    if (t >= 0xcc && t <= 0xcf) { p++; *v = be(1 << (t - 0xcc)); return ok; }
    if (t >= 0xd0 && t <= 0xd3) { p++; *v = be(1 << (t - 0xd0)); return ok; }
    return false;
  }
  bool container(uint8_t fix_lo, uint8_t t16, size_t* n) {     // map or array header
    if (p >= e) return ok = false;
    uint8_t t = *p;
    if (t >= fix_lo && t <= fix_lo + 0x0f) { *n = t & 0x0f; p++; return true; }
    if (t == t16) { p++; *n = (size_t)be(2); return ok; }
    if (t == t16 + 1) { p++; *n = (size_t)be(4); return ok; }
    return false;
  }
  bool map(size_t* n) { return container(0x80, 0xde, n); }
  bool array(size_t* n) { return container(0x90, 0xdc, n); }
  void skip(int depth = 0) {
    if (!ok || p >= e || depth > 64) { ok = false; return; }
    size_t n;
    const char* s;
    uint64_t v;
    uint8_t t = *p;
    if (map(&n)) { for (size_t i = 0; i < 2 * n && ok; i++) skip(depth + 1); return; }
    if (array(&n)) { for (size_t i = 0; i < n && ok; i++) skip(depth + 1); return; }
    if (str(&s, &n) || uint_(&v)) return;
    if (!ok) return;
    p++;
    if (t == 0xc0 || t == 0xc2 || t == 0xc3 || t >= 0xe0) return;                 // nil, bool, negative fixint
    if (t == 0xca) { be(4); return; }
    if (t == 0xcb) { be(8); return; }
    if (t >= 0xc4 && t <= 0xc6) { size_t len = (size_t)be(1 << (t - 0xc4)); if ((size_t)(e - p) < len) ok = false; else p += len; return; }
    if (t >= 0xd4 && t <= 0xd8) { be(1 + (1 << (t - 0xd4))); return; }           // fixext
    if (t >= 0xc7 && t <= 0xc9) { size_t len = (size_t)be(1 << (t - 0xc7)); be(1); if ((size_t)(e - p) < len) ok = false; else p += len; return; }
    ok = false;
  }
};

bool key_is(const char* s, size_t n, const char* lit) { return n == strlen(lit) && memcmp(s, lit, n) == 0; }

// Bytes of the explicit arguments of `kernel` (the end of its last argument that is not one of the
// hidden ones the runtime appends, e.g. the grid size) from an AMDGPU metadata blob; 0 when not found.
// Falls back to the whole argument segment for a kernel whose metadata lists no arguments.
size_t kernarg_from_metadata(const uint8_t* d, size_t len, const char* kernel) {
  MsgPack m{d, d + len};
  size_t n;
  if (!m.map(&n)) return 0;
  for (size_t i = 0; i < n && m.ok; i++) {
    const char* k; size_t kn;
    if (!m.str(&k, &kn)) return 0;
    if (!key_is(k, kn, "amdhsa.kernels")) { m.skip(); continue; }
    size_t nk;
    if (!m.array(&nk)) return 0;
    for (size_t j = 0; j < nk && m.ok; j++) {
      size_t nf;
      if (!m.map(&nf)) return 0;
      bool mine = false, has_args = false;
      uint64_t segment = 0, explicit_end = 0;
      for (size_t f = 0; f < nf && m.ok; f++) {
        const char* fk; size_t fkn;
        if (!m.str(&fk, &fkn)) return 0;
        if (key_is(fk, fkn, ".name")) {
          const char* v; size_t vn;
          if (!m.str(&v, &vn)) return 0;
          mine = key_is(v, vn, kernel);
        } else if (key_is(fk, fkn, ".kernarg_segment_size")) {
          if (!m.uint_(&segment)) return 0;
        } else if (key_is(fk, fkn, ".args")) {
          size_t na;
          if (!m.array(&na)) return 0;
          has_args = true;
          for (size_t a = 0; a < na && m.ok; a++) {
            size_t nq;
            if (!m.map(&nq)) return 0;
            uint64_t off = 0, size = 0;
            bool hidden = false;
            for (size_t q = 0; q < nq && m.ok; q++) {
              const char* ak; size_t akn;
              if (!m.str(&ak, &akn)) return 0;
              if (key_is(ak, akn, ".offset")) { if (!m.uint_(&off)) return 0; }
              else if (key_is(ak, akn, ".size")) { if (!m.uint_(&size)) return 0; }
              else if (key_is(ak, akn, ".value_kind")) {
                const char* v; size_t vn;
                if (!m.str(&v, &vn)) return 0;
                hidden = vn >= 7 && memcmp(v, "hidden_", 7) == 0;
              } else m.skip();
            }
            if (!hidden && off + size > explicit_end) explicit_end = off + size;
          }
        } else {
          m.skip();
        }
      }
      if (mine && m.ok) return (size_t)(has_args ? ((explicit_end + 7) & ~(uint64_t)7) : segment);
    }
    return 0;
  }
  return 0;
}

// The gfx ELF inside `image` (an ELF itself, or an uncompressed clang offload bundle holding one).
bool find_device_elf(const std::vector<char>& image, const uint8_t** elf, size_t* len) {
  const uint8_t* b = (const uint8_t*)image.data();
  size_t n = image.size();
  static const char kBundle[] = "__CLANG_OFFLOAD_BUNDLE__";
  if (n > 64 && memcmp(b, "\177ELF", 4) == 0) { *elf = b; *len = n; return true; }
  if (n < 32 || memcmp(b, kBundle, sizeof kBundle - 1) != 0) return false;
  uint64_t count;
  memcpy(&count, b + 24, 8);
  size_t off = 32;
  for (uint64_t i = 0; i < count && i < 64; i++) {
    if (off + 24 > n) return false;
    uint64_t eo, es, tl;
    memcpy(&eo, b + off, 8); memcpy(&es, b + off + 8, 8); memcpy(&tl, b + off + 16, 8);
    off += 24;
    if (tl > n || off + tl > n) return false;
    bool device = tl >= 3 && memcmp(b + off, "hip", 3) == 0;
    off += tl;
    if (device && es > 64 && eo <= n && es <= n - eo && memcmp(b + eo, "\177ELF", 4) == 0) { *elf = b + eo; *len = (size_t)es; return true; }
  }
  return false;
}

// 0 when the image has no readable metadata for `kernel` (the launch check is then skipped)
size_t explicit_arg_bytes(const std::vector<char>& image, const char* kernel) {
  const uint8_t* e; size_t n;
  if (!find_device_elf(image, &e, &n) || n < 64 || e[4] != 2 /*ELFCLASS64*/ || e[5] != 1 /*little endian*/) return 0;
  uint64_t shoff; uint16_t shentsize, shnum;
  memcpy(&shoff, e + 0x28, 8); memcpy(&shentsize, e + 0x3a, 2); memcpy(&shnum, e + 0x3c, 2);
  if (shentsize < 64 || shoff > n || (uint64_t)shnum * shentsize > n - shoff) return 0;
  for (unsigned i = 0; i < shnum; i++) {
    const uint8_t* sh = e + shoff + (uint64_t)i * shentsize;
    uint32_t type; uint64_t off, size;
    memcpy(&type, sh + 4, 4); memcpy(&off, sh + 0x18, 8); memcpy(&size, sh + 0x20, 8);
    if (type != 7 /*SHT_NOTE*/ || off > n || size > n - off) continue;
    const uint8_t* p = e + off; const uint8_t* end = p + size;
    while ((size_t)(end - p) >= 12) {
      uint32_t namesz, descsz, ntype;
      memcpy(&namesz, p, 4); memcpy(&descsz, p + 4, 4); memcpy(&ntype, p + 8, 4);
      p += 12;
      size_t na = ((size_t)namesz + 3) & ~(size_t)3, da = ((size_t)descsz + 3) & ~(size_t)3;
      if (na > (size_t)(end - p) || da > (size_t)(end - p) - na) break;
      if (ntype == 32 /*NT_AMDGPU_METADATA*/ && namesz == 7 && memcmp(p, "AMDGPU", 6) == 0) {
        size_t r = kernarg_from_metadata(p + na, descsz, kernel);
        if (r) return r;
      }
      p += na + da;
    }
  }
  return 0;
}

}  // namespace

extern "C" {

int frnn_version(void) { return 100; }

const char* frnn_last_error(void) { return g_err.c_str(); }

int frnn_compile(const char* src, size_t len, const char* arch, const char* opts,
                 const char* cache_dir, const char* key, char* out_path, size_t cap) {
  if (!src || !arch || !cache_dir || !key || !out_path || cap == 0)
    return fail(FRNN_ERR_ARG, "frnn_compile: null argument");
  for (const char* p = key; *p; p++)
    if (!((*p >= 'a' && *p <= 'z') || (*p >= 'A' && *p <= 'Z') || (*p >= '0' && *p <= '9') || *p == '_' || *p == '-'))
      return fail(FRNN_ERR_ARG, "frnn_compile: key may only hold [A-Za-z0-9_-]");
  std::string dir(cache_dir);
  if (mkdirs(dir) != 0) return fail(FRNN_ERR_IO, "cannot create cache directory %s: %s", cache_dir, strerror(errno));
  std::string base = dir + "/" + key;
  std::string hsaco = base + ".hsaco";
  if (hsaco.size() + 1 > cap) return fail(FRNN_ERR_ARG, "frnn_compile: out_path too small");
  strcpy(out_path, hsaco.c_str());
  if (file_exists(hsaco)) return FRNN_OK;

  // serialise concurrent builders of the same key
  std::string lockp = base + ".lock";
  int lockfd = open(lockp.c_str(), O_CREAT | O_RDWR, 0666);
  if (lockfd < 0) return fail(FRNN_ERR_IO, "cannot open lock file %s: %s", lockp.c_str(), strerror(errno));
  if (flock(lockfd, LOCK_EX) != 0) {
    close(lockfd);
    return fail(FRNN_ERR_IO, "cannot lock %s: %s", lockp.c_str(), strerror(errno));
  }
  struct Unlock {
    int fd;
    ~Unlock() { flock(fd, LOCK_UN); close(fd); }
  } unlock{lockfd};
  if (file_exists(hsaco)) return FRNN_OK;   // someone else built it while we waited

  std::string srcp = base + ".hip";
  if (write_file(srcp, src, len) != 0) return fail(FRNN_ERR_IO, "cannot write %s: %s", srcp.c_str(), strerror(errno));
  char tmpn[64];
  snprintf(tmpn, sizeof tmpn, ".tmp%d", (int)getpid());
  std::string tmpo = hsaco + tmpn;
  std::string logp = base + ".log";

  std::vector<std::string> av = {find_hipcc(), "--genco", std::string("--offload-arch=") + arch, "-O3", "-std=c++17",
                                 // packed fp32 VALU ops are kept off on this hardware pool
                                 "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  for (auto& o : split_ws(opts)) av.push_back(o);
  av.push_back("-o");
  av.push_back(tmpo);
  av.push_back(srcp);
  std::vector<char*> argv;
  for (auto& s : av) argv.push_back(const_cast<char*>(s.c_str()));
  argv.push_back(nullptr);

  posix_spawn_file_actions_t fa;
  posix_spawn_file_actions_init(&fa);
  posix_spawn_file_actions_addopen(&fa, 1, logp.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0666);
  posix_spawn_file_actions_adddup2(&fa, 1, 2);
  pid_t pid;
  int rc = posix_spawnp(&pid, argv[0], &fa, nullptr, argv.data(), environ);
  posix_spawn_file_actions_destroy(&fa);
  if (rc != 0) return fail(FRNN_ERR_COMPILE, "cannot start %s: %s", argv[0], strerror(rc));
  int status = 0;
  while (waitpid(pid, &status, 0) < 0) {
    if (errno != EINTR) return fail(FRNN_ERR_COMPILE, "waitpid failed: %s", strerror(errno));
  }
  if (!WIFEXITED(status) || WEXITSTATUS(status) != 0 || !file_exists(tmpo)) {
    std::string log = read_tail(logp, 3000);
    unlink(tmpo.c_str());
    return fail(FRNN_ERR_COMPILE, "hipcc failed (status %d) for %s:\n%s", status, srcp.c_str(), log.c_str());
  }
  if (rename(tmpo.c_str(), hsaco.c_str()) != 0) {
    unlink(tmpo.c_str());
    return fail(FRNN_ERR_IO, "cannot rename %s: %s", tmpo.c_str(), strerror(errno));
  }
  return FRNN_OK;
}

int frnn_module_load(const char* path, frnn_module_t* out) {
  if (!path || !out) return fail(FRNN_ERR_ARG, "frnn_module_load: null argument");
  HipApi& h = hip();
  if (!h.ok) return fail(FRNN_ERR_NO_HIP, "%s", h.why.c_str());
  // The image is read here and handed over in memory: the file may be replaced by a rebuild
  // later, and the module must not depend on it.
  FILE* f = fopen(path, "rb");
  if (!f) return fail(FRNN_ERR_IO, "cannot open code object %s: %s", path, strerror(errno));
  fseek(f, 0, SEEK_END);
  long n = ftell(f);
  fseek(f, 0, SEEK_SET);
  frnn_module_s* m = new frnn_module_s{nullptr, std::vector<char>((size_t)(n > 0 ? n : 0)), {}};
  size_t got = n > 0 ? fread(m->image.data(), 1, (size_t)n, f) : 0;
  fclose(f);
  if (n <= 0 || got != (size_t)n) {
    delete m;
    return fail(FRNN_ERR_IO, "cannot read code object %s", path);
  }
  // refuse anything that is not an offload bundle or an ELF image before the driver parses it
  static const char kBundle[] = "__CLANG_OFFLOAD_BUNDLE__";
  bool bundle = (size_t)n > sizeof kBundle && memcmp(m->image.data(), kBundle, sizeof kBundle - 1) == 0;
  bool elf = n > 64 && memcmp(m->image.data(), "\177ELF", 4) == 0;
  if (!bundle && !elf) {
    delete m;
    return fail(FRNN_ERR_IO, "%s is not a code object (damaged cache entry?)", path);
  }
  hipError_t e = h.ModuleLoadData(&m->mod, m->image.data());
  if (e != 0) {
    delete m;
    return hip_fail("hipModuleLoadData", e);
  }
  *out = m;
  return FRNN_OK;
}

int frnn_get_kernel(frnn_module_t m, const char* name, frnn_kernel_t* out) {
  if (!m || !name || !out) return fail(FRNN_ERR_ARG, "frnn_get_kernel: null argument");
  HipApi& h = hip();
  if (!h.ok) return fail(FRNN_ERR_NO_HIP, "%s", h.why.c_str());
  void* fn = nullptr;
  hipError_t e = h.ModuleGetFunction(&fn, m->mod, name);
  if (e != 0) return hip_fail("hipModuleGetFunction", e);
  frnn_kernel_s* k = new frnn_kernel_s{fn, explicit_arg_bytes(m->image, name)};
  {
    std::lock_guard<std::mutex> lock(m->mu);      // (threads may fetch kernels of one module side by side)
    m->kernels.push_back(k);
  }
  *out = k;
  return FRNN_OK;
}

void* frnn_detail_runtime_launch_symbol() {
  HipApi& h = hip();
  return h.ok ? (void*)h.ModuleLaunchKernel : nullptr;
}

int frnn_kernel_arg_bytes(frnn_kernel_t k, size_t* out) {
  if (!k || !out) return fail(FRNN_ERR_ARG, "frnn_kernel_arg_bytes: null argument");
  *out = k->kernarg;
  return FRNN_OK;
}

int frnn_launch(frnn_kernel_t k, const uint32_t grid[3], const uint32_t block[3],
                uint32_t lds_bytes, void* stream, const void* args, size_t arg_bytes) {
  if (!k || !grid || !block || (!args && arg_bytes)) return fail(FRNN_ERR_ARG, "frnn_launch: null argument");
  for (int i = 0; i < 3; i++)
    if (grid[i] == 0 || block[i] == 0) return fail(FRNN_ERR_ARG, "frnn_launch: empty grid or block");
  if ((uint64_t)block[0] * block[1] * block[2] > 1024) return fail(FRNN_ERR_ARG, "frnn_launch: block larger than 1024 threads");
  if (grid[1] > 65535 || grid[2] > 65535) return fail(FRNN_ERR_ARG, "frnn_launch: grid y/z larger than 65535");
  HipApi& h = hip();
  if (!h.ok) return fail(FRNN_ERR_NO_HIP, "%s", h.why.c_str());
  // The block must be exactly as large as the kernel's explicit kernarg segment; kernels of
  // this project take 8-byte fields only, so anything else is a packing mistake (a short block
  // leaves the kernel reading arguments that were never set).
  if (arg_bytes % 8 != 0) return fail(FRNN_ERR_ARG, "frnn_launch: argument block must be a whole number of 8-byte words");
  if (k->kernarg && arg_bytes != k->kernarg)
    return fail(FRNN_ERR_ARG, "frnn_launch: argument block of %zu bytes, the kernel's code object declares %zu", arg_bytes, k->kernarg);
  size_t sz = arg_bytes;
  void* extra[] = {(void*)0x01 /*BUFFER_POINTER*/, const_cast<void*>(args), (void*)0x02 /*BUFFER_SIZE*/, &sz,
                   (void*)0x03 /*END*/};
  hipError_t e = h.ModuleLaunchKernel(k->fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds_bytes, stream,
                                      nullptr, extra);
  if (e != 0) return hip_fail("hipModuleLaunchKernel", e);
  return FRNN_OK;
}

int frnn_module_free(frnn_module_t m) {
  if (!m) return FRNN_OK;
  HipApi& h = hip();
  hipError_t e = 0;
  if (h.ok && m->mod) e = h.ModuleUnload(m->mod);
  for (frnn_kernel_s* k : m->kernels) delete k;
  delete m;
  if (e != 0) return hip_fail("hipModuleUnload", e);
  return FRNN_OK;
}

int frnn_device_cus(void) {
  HipApi& h = hip();
  if (!h.ok) return -1;
  int dev = 0, cus = 0;
  if (h.GetDevice(&dev) != 0) return -1;
  if (h.DeviceGetAttribute(&cus, 63 /*hipDeviceAttributeMultiprocessorCount*/, dev) != 0) return -1;
  return cus;
}

}  // extern "C"
