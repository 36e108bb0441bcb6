// hipsim: run an emitted HIP kernel on the CPU, one workgroup at a time.  TEST TOOL ONLY.
//
// Every GPU thread of a workgroup is a ucontext fiber on one OS thread.  A barrier yields to
// the scheduler, which resumes the fibers round-robin, so "resume every fiber once" is one
// barrier phase.  Cross-lane operations (DPP, shuffles) are an exchange through a per-block
// array bracketed by two such barriers, which is valid because the kernels only reduce in
// workgroup-uniform control flow.  `__shared__` becomes `static` (workgroups run one after
// another).  Buffers handed to the kernel come from sim_alloc(), which places them against a
// PROT_NONE guard page, so an out-of-bounds access ends the process with SIGSEGV instead of
// passing silently.
#pragma once
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <ucontext.h>
#include <unistd.h>

#include <algorithm>
#include <functional>
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

static int sim_run_grid(const std::function<void()>& body, int gx, int gy, int gz, int bx) {
  const size_t STACK = 256 * 1024;
  std::vector<char*> stacks(bx);
  for (int i = 0; i < bx; i++) stacks[i] = (char*)malloc(STACK);
  sim_body = body;
  blockDim = {(unsigned)bx, 1, 1};
  gridDim = {(unsigned)gx, (unsigned)gy, (unsigned)gz};
  for (int bz = 0; bz < gz; bz++)
    for (int by = 0; by < gy; by++)
      for (int bxi = 0; bxi < gx; bxi++) {
        blockIdx = {(unsigned)bxi, (unsigned)by, (unsigned)bz};
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
          for (int i = 0; i < bx; i++) {
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

template <class T> static inline T __hip_atomic_fetch_add(T* p, T v, int, int) {
  T o = *p;
  *p = o + v;
  return o;
}

// ------------------------------------------------------------------ math + narrow floats
#define __expf(x) expf(x)
#define __builtin_amdgcn_exp2f(x) exp2f(x)
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
#include <map>
static std::map<void*, std::pair<void*, size_t>> sim_maps;

// `nbytes` of read/write memory with an inaccessible page on both sides.  With `against_end`
// the block ends (up to 16-byte alignment) at the trailing guard page, otherwise it starts
// right after the leading one.
extern "C" void* sim_alloc(size_t nbytes, int against_end) {
  size_t page = (size_t)sysconf(_SC_PAGESIZE);
  size_t body = (nbytes + page - 1) / page * page;
  if (body == 0) body = page;
  char* base = (char*)mmap(nullptr, body + 2 * page, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0);
  if (base == MAP_FAILED) return nullptr;
  mprotect(base, page, PROT_NONE);
  mprotect(base + page + body, page, PROT_NONE);
  char* p = base + page;
  if (against_end) p += (body - nbytes) & ~(size_t)15;
  sim_maps[p] = {base, body + 2 * page};
  return p;
}

extern "C" void sim_free(void* p) {
  auto it = sim_maps.find(p);
  if (it == sim_maps.end()) return;
  munmap(it->second.first, it->second.second);
  sim_maps.erase(it);
}
