// hipsim: run an emitted HIP kernel on the CPU, one workgroup at a time.  TEST TOOL ONLY.
//
// Every GPU thread of a workgroup is a ucontext fiber on one OS thread.  A barrier yields to
// the scheduler, which resumes every fiber once per barrier phase: in index order, or - with
// HIPSIM_SEED set to a non-zero number - in a fresh random order in every phase, with the
// workgroups of the grid shuffled as well, so that code which only works for one order of the
// threads between two barriers (a missing barrier, a read of LDS before its write) or of the
// workgroups gives wrong results for some seed.  Cross-lane operations (DPP, shuffles) are an
// exchange through a per-block array bracketed by two such barriers, which is valid because the
// kernels only reduce in workgroup-uniform control flow.  `__shared__` becomes `static`
// (workgroups run one after another); the harness's build step adds a call of sim_lds_poison()
// after every such declaration, which fills the array with NaNs when a workgroup first reaches
// it: LDS holds no zeros at the start of a workgroup and keeps nothing from the one before.
// Buffers handed to the kernel come from sim_alloc(), which places them between two
// inaccessible regions of SIM_GUARD bytes each, so an access outside a tensor - by less than that -
// ends the process with SIGSEGV (the handler names the address, the nearest tensor, block and thread)
// instead of passing silently.
#pragma once
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <ucontext.h>
#include <unistd.h>

#include <signal.h>

#include <algorithm>
#include <functional>
#include <map>
#include <random>
#include <vector>

struct sim_dim3 { unsigned x, y, z; };
static sim_dim3 threadIdx, blockIdx, blockDim, gridDim;

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline
#define __shared__ static
#define __launch_bounds__(...)
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __builtin_amdgcn_sched_barrier(mask) ((void)0)      // (a hint to the GPU compiler's scheduler)
using std::max;
using std::min;

// ------------------------------------------------------------------ fibers + barrier
static ucontext_t sim_sched_ctx;
static std::vector<ucontext_t> sim_fibers;
static std::vector<char> sim_done;
static int sim_cur = -1;
static std::function<void()> sim_body;

static void sim_trampoline() {
  sim_body();
  sim_done[sim_cur] = 1;
  swapcontext(&sim_fibers[sim_cur], &sim_sched_ctx);
}

static inline void sim_barrier() {
  int me = sim_cur;
  swapcontext(&sim_fibers[me], &sim_sched_ctx);
  threadIdx.x = (unsigned)me;
}
#define __syncthreads() sim_barrier()

static unsigned long sim_block_epoch = 0;      // counts workgroups; LDS arrays are poisoned once per workgroup
static size_t sim_lds_bytes = 0, sim_lds_peak = 0;

// Called right after the declaration of a `__shared__` array: the first thread of a workgroup that gets
// there fills it with NaNs (what a workgroup finds in LDS is undefined) and counts its size.
static inline void sim_lds_poison(void* p, size_t nbytes) {
  static std::map<void*, unsigned long> seen;
  unsigned long& e = seen[p];
  if (e == sim_block_epoch) return;
  e = sim_block_epoch;
  uint32_t* w = (uint32_t*)p;
  for (size_t i = 0; i < nbytes / 4; i++) w[i] = 0x7fc0dead;
  sim_lds_bytes += nbytes;
  sim_lds_peak = std::max(sim_lds_peak, sim_lds_bytes);
}
extern "C" size_t sim_lds_peak_bytes() { return sim_lds_peak; }

static int sim_run_grid(const std::function<void()>& body, int gx, int gy, int gz, int bx) {
  const size_t STACK = 256 * 1024;
  const char* seed_env = getenv("HIPSIM_SEED");
  const unsigned long seed = seed_env ? strtoul(seed_env, nullptr, 10) : 0;
  std::mt19937 rng((unsigned)seed);
  std::vector<char*> stacks(bx);
  for (int i = 0; i < bx; i++) stacks[i] = (char*)malloc(STACK);
  sim_body = body;
  blockDim = {(unsigned)bx, 1, 1};
  gridDim = {(unsigned)gx, (unsigned)gy, (unsigned)gz};
  std::vector<long> blocks((size_t)gx * gy * gz);
  for (size_t i = 0; i < blocks.size(); i++) blocks[i] = (long)i;
  if (seed) std::shuffle(blocks.begin(), blocks.end(), rng);
  std::vector<int> order(bx);
  for (long blk : blocks) {
    blockIdx = {(unsigned)(blk % gx), (unsigned)((blk / gx) % gy), (unsigned)(blk / ((long)gx * gy))};
    sim_block_epoch++;
    sim_lds_bytes = 0;
    sim_fibers.assign(bx, ucontext_t());
    sim_done.assign(bx, 0);
    for (int i = 0; i < bx; i++) {
      getcontext(&sim_fibers[i]);
      sim_fibers[i].uc_stack.ss_sp = stacks[i];
      sim_fibers[i].uc_stack.ss_size = STACK;
      sim_fibers[i].uc_link = &sim_sched_ctx;
      makecontext(&sim_fibers[i], sim_trampoline, 0);
    }
    int remaining = bx;
    while (remaining > 0) {
      int finished_now = 0, alive = 0;
      for (int i = 0; i < bx; i++) order[i] = i;
      if (seed) std::shuffle(order.begin(), order.end(), rng);
      for (int k = 0; k < bx; k++) {
        const int i = order[k];
        if (sim_done[i]) continue;
        alive++;
        sim_cur = i;
        threadIdx = {(unsigned)i, 0, 0};
        swapcontext(&sim_sched_ctx, &sim_fibers[i]);
        if (sim_done[i]) finished_now++;
      }
      // all threads of a workgroup must leave together (no early exit before a barrier)
      if (finished_now != 0 && finished_now != alive) {
        fprintf(stderr, "hipsim: threads of one workgroup ended at different barriers\n");
        return 1;
      }
      remaining -= finished_now;
    }
  }
  for (int i = 0; i < bx; i++) free(stacks[i]);
  return 0;
}

// ------------------------------------------------------------------ cross-lane ops
static int sim_xchg[1024];

static inline int sim_lane_read(int v, int src_lane_in_wave) {
  int t = (int)threadIdx.x, base = t & ~63;
  sim_xchg[t] = v;
  sim_barrier();
  int r = sim_xchg[base + src_lane_in_wave];
  sim_barrier();
  return r;
}

static inline int __builtin_amdgcn_update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
  (void)old; (void)bound_ctrl;
  if (row_mask != 0xf || bank_mask != 0xf) { fprintf(stderr, "hipsim: dpp masks unsupported\n"); abort(); }
  int lane = (int)threadIdx.x & 63, s;
  if (ctrl >= 0 && ctrl <= 0xff) s = (lane & ~3) + ((ctrl >> (2 * (lane & 3))) & 3);   // quad_perm
  else if (ctrl == 0x140) s = (lane & ~15) + 15 - (lane & 15);                           // row_mirror
  else if (ctrl == 0x141) s = (lane & ~7) + 7 - (lane & 7);                              // row_half_mirror
  else { fprintf(stderr, "hipsim: dpp ctrl 0x%x unsupported\n", ctrl); abort(); }
  return sim_lane_read(src, s);
}

static inline int __builtin_amdgcn_readfirstlane(int v) { return sim_lane_read(v, 0); }

// gfx950 row swaps.  Both return the pair (new first operand, new second operand).
// permlane16_swap exchanges the odd 16-lane rows of the first operand with the even rows of the
// second: first' = [a.row0, b.row0, a.row2, b.row2], second' = [a.row1, b.row1, a.row3, b.row3].
// permlane32_swap does the same with the 32-lane halves: first' = [a.lo, b.lo], second' = [a.hi, b.hi].
struct sim_u2 {
  unsigned v[2];
  unsigned operator[](int i) const { return v[i]; }
};
static inline sim_u2 sim_permlane_swap(unsigned a, unsigned b, int width) {
  const int lane = (int)threadIdx.x & 63;
  const bool upper = (lane / width) & 1;                   // an odd row (the upper half)
  const unsigned a_far = (unsigned)sim_lane_read((int)a, lane ^ width);
  const unsigned b_far = (unsigned)sim_lane_read((int)b, lane ^ width);
  sim_u2 r;
  r.v[0] = upper ? b_far : a;       // odd rows of the first operand take the second operand's even rows
  r.v[1] = upper ? b : a_far;       // even rows of the second operand take the first operand's odd rows
  return r;
}
static inline sim_u2 __builtin_amdgcn_permlane16_swap(unsigned a, unsigned b, bool, bool) { return sim_permlane_swap(a, b, 16); }
static inline sim_u2 __builtin_amdgcn_permlane32_swap(unsigned a, unsigned b, bool, bool) { return sim_permlane_swap(a, b, 32); }

static inline float __shfl_xor(float v, int mask, int width = 64) {
  (void)width;
  int i;
  memcpy(&i, &v, 4);
  int r = sim_lane_read(i, ((int)threadIdx.x & 63) ^ mask);
  float f;
  memcpy(&f, &r, 4);
  return f;
}

// (a macro, not a function of that name: clang knows the name as a builtin)
template <class T> static inline T sim_atomic_fetch_add(T* p, T v, int, int) {
  T o = *p;
  *p = o + v;
  return o;
}
#define __hip_atomic_fetch_add sim_atomic_fetch_add

// ------------------------------------------------------------------ math + narrow floats
#define __expf(x) expf(x)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_rcpf(x) (1.0f / (x))
#define __logf(x) logf(x)
#define __log2f(x) log2f(x)
static inline float rsqrtf(float x) { return 1.0f / sqrtf(x); }

struct sim_bf16 {
  uint16_t bits;
  sim_bf16() : bits(0) {}
  explicit sim_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) { bits = 0x7fc0; return; }
    u += 0x7fffu + ((u >> 16) & 1u);
    bits = (uint16_t)(u >> 16);
  }
};
#define __bf16 sim_bf16

struct sim_half {
  uint16_t bits;
  sim_half() : bits(0) {}
  explicit sim_half(float f) {            // round to nearest even
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u, mant = x & 0x7fffffu;
    int exp = (int)((x >> 23) & 0xff) - 127 + 15;
    if (((x >> 23) & 0xff) == 0xff) { bits = (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0)); return; }
    if (exp >= 31) { bits = (uint16_t)(sign | 0x7c00u); return; }
    if (exp <= 0) {
      if (exp < -10) { bits = (uint16_t)sign; return; }
      mant |= 0x800000u;
      int shift = 14 - exp;
      uint32_t h = mant >> shift, rem = mant & ((1u << shift) - 1), half = 1u << (shift - 1);
      if (rem > half || (rem == half && (h & 1))) h++;
      bits = (uint16_t)(sign | h);
      return;
    }
    uint32_t h = ((uint32_t)exp << 10) | (mant >> 13), rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) h++;
    bits = (uint16_t)(sign | h);
  }
  explicit operator float() const {
    uint32_t sign = (uint32_t)(bits & 0x8000u) << 16, exp = (bits >> 10) & 0x1f, mant = bits & 0x3ffu, u;
    if (exp == 0) {
      if (mant == 0) u = sign;
      else {
        int e = -1;
        do { mant <<= 1; e++; } while (!(mant & 0x400u));
        u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
      }
    } else if (exp == 31) u = sign | 0x7f800000u | (mant << 13);
    else u = sign | ((exp - 15 + 127) << 23) | (mant << 13);
    float f;
    memcpy(&f, &u, 4);
    return f;
  }
};
#define _Float16 sim_half

// ------------------------------------------------------------------ guarded allocation
static std::map<void*, std::pair<void*, size_t>> sim_maps;

// `nbytes` of read/write memory with SIM_GUARD inaccessible bytes on both sides (address space only).  With
// `against_end` the block ends (up to 16-byte alignment) at the trailing guard, otherwise it starts right
// after the leading one.
static const size_t SIM_GUARD = (size_t)1 << 30;
struct sim_block_info { char* lo; size_t nbytes; };
static std::vector<sim_block_info> sim_live;

static void sim_segv(int, siginfo_t* si, void*) {
  char* a = (char*)si->si_addr;
  fprintf(stderr, "hipsim: access outside every tensor at %p, block (%u,%u,%u) thread %u\n", (void*)a, blockIdx.x, blockIdx.y,
          blockIdx.z, threadIdx.x);
  for (size_t i = 0; i < sim_live.size(); i++) {
    long before = (long)(sim_live[i].lo - a), after = (long)(a - (sim_live[i].lo + sim_live[i].nbytes));
    if (before > 0 && before <= (long)SIM_GUARD) fprintf(stderr, "  %ld bytes before tensor #%zu (%zu bytes)\n", before, i, sim_live[i].nbytes);
    if (after >= 0 && after < (long)SIM_GUARD) fprintf(stderr, "  %ld bytes past the end of tensor #%zu (%zu bytes)\n", after, i, sim_live[i].nbytes);
  }
  _exit(139);
}

extern "C" void* sim_alloc(size_t nbytes, int against_end) {
  static bool handler = false;
  if (!handler) {
    handler = true;
    static char altstack[64 * 1024];
    stack_t ss = {altstack, 0, sizeof(altstack)};
    sigaltstack(&ss, nullptr);
    struct sigaction sa;
    memset(&sa, 0, sizeof(sa));
    sa.sa_sigaction = sim_segv;
    sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
    sigaction(SIGSEGV, &sa, nullptr);
  }
  size_t page = (size_t)sysconf(_SC_PAGESIZE);
  size_t body = (nbytes + page - 1) / page * page;
  if (body == 0) body = page;
  char* base = (char*)mmap(nullptr, body + 2 * SIM_GUARD, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
  if (base == MAP_FAILED) return nullptr;
  mprotect(base + SIM_GUARD, body, PROT_READ | PROT_WRITE);
  char* p = base + SIM_GUARD;
  if (against_end) p += (body - nbytes) & ~(size_t)15;
  sim_maps[p] = {base, body + 2 * SIM_GUARD};
  sim_live.push_back({p, nbytes});
  return p;
}

extern "C" void sim_free(void* p) {
  auto it = sim_maps.find(p);
  if (it == sim_maps.end()) return;
  munmap(it->second.first, it->second.second);
  sim_maps.erase(it);
  for (size_t i = 0; i < sim_live.size(); i++)
    if (sim_live[i].lo == (char*)p) { sim_live.erase(sim_live.begin() + i); break; }
}
