/* frnn_rt - C ABI of the MI355X kernel runtime behind flex_rnn's generated kernels.
 *
 * This is the seam where the reference hands generated source to a compiler and gets
 * launchable callables back: `build_cuda(*(src, grid, threads)) -> callables`
 * (/root/reference/flex_rnn/to_cuda.py:230-280), which writes the source under a cache
 * directory keyed by its md5 (to_cuda.py:264, 274-276), builds it with nvcc through
 * torch.utils.cpp_extension.load (to_cuda.py:279) and launches each kernel as
 * `k<<<grid, threads>>>(ptrs...)` on the default stream with no error check
 * (to_cuda.py:245-247).
 *
 * Here the same steps are plain C entry points: compile HIP source for gfx950 into an
 * on-disk code-object cache, load a code object, look a kernel up, launch it on a caller
 * supplied stream with a packed argument buffer.  All functions return 0 on success and a
 * non-zero code on failure; `frnn_last_error()` then returns a thread-local message.  No
 * function synchronises the device or allocates device memory; all device buffers are owned
 * by the caller.  The library binds to the HIP runtime already loaded in the process (the
 * one PyTorch ships) and never loads a second one if one is present.
 */
#ifndef FRNN_RT_H
#define FRNN_RT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct frnn_module_s* frnn_module_t;   /* opaque: a loaded code object            */
typedef struct frnn_kernel_s* frnn_kernel_t;   /* opaque: a kernel inside a loaded module */

enum {
  FRNN_OK = 0,
  FRNN_ERR_ARG = 1,        /* bad argument                                   */
  FRNN_ERR_IO = 2,         /* cache directory / file problem                  */
  FRNN_ERR_COMPILE = 3,    /* hipcc failed; message holds the compiler output */
  FRNN_ERR_NO_HIP = 4,     /* no HIP runtime / no device                      */
  FRNN_ERR_HIP = 5         /* a HIP call failed; message holds its name+code  */
};

/* Library version, major*100+minor.  Replaces nothing in the reference (it has no runtime). */
int frnn_version(void);

/* Message for the last failure on the calling thread ("" if none). */
const char* frnn_last_error(void);

/* Compile `src` (HIP C++, `len` bytes) for `arch` (e.g. "gfx950") with extra hipcc options
 * `opts` (may be NULL) into `<cache_dir>/<key>.hsaco`, unless that file already exists.
 * The source is kept beside it as `<key>.hip`.  Concurrent callers are serialised with a
 * lock file and the code object appears atomically (rename).  Writes the code-object path
 * into `out_path` (capacity `cap`).  Needs no GPU.
 * Replaces: to_cuda.py:264-279 (md5-named files under /tmp/flex_rnn + cpp_extension.load). */
int frnn_compile(const char* src, size_t len, const char* arch, const char* opts,
                 const char* cache_dir, const char* key, char* out_path, size_t cap);

/* Load a code object file into the current device's context.  The file is read into memory
 * owned by the module (hipModuleLoadData), so it may be rebuilt or removed afterwards; a file
 * that is neither an offload bundle nor an ELF image is rejected with FRNN_ERR_IO.
 * Replaces: the dlopen done by cpp_extension.load (to_cuda.py:279). */
int frnn_module_load(const char* path, frnn_module_t* out);

/* Look up an `extern "C" __global__` kernel by name.
 * Replaces: getattr(torch.ops.<id>, func_name) (to_cuda.py:280). */
int frnn_get_kernel(frnn_module_t m, const char* name, frnn_kernel_t* out);

/* Size in bytes of the kernel's explicit arguments as recorded in its code object (the `.args` of
 * the AMDGPU metadata note up to the end of the last argument that is not a hidden one, rounded up
 * to 8), or 0 when the image carries no readable metadata.  `frnn_launch` rejects a block of any
 * other size.
 * Replaces: the typed C++ launcher the reference generates per kernel (to_cuda.py:236-247), where the
 * compiler checks the argument list. */
int frnn_kernel_arg_bytes(frnn_kernel_t k, size_t* out);

/* Launch `k` with the given grid (in workgroups) and block (in threads) on `stream`
 * (a hipStream_t; NULL = default stream).  `args` points to `arg_bytes` bytes laid out
 * exactly as the kernel's parameter list (one by-value struct of 8-byte fields in this
 * project).  `arg_bytes` must equal the size of that parameter list (checked against the code
 * object's metadata, see frnn_kernel_arg_bytes) and be a multiple of 8; a shorter block would
 * leave the kernel with unset arguments.  Returns after enqueueing;
 * stream-ordered, never synchronises.
 * Replaces: the generated `k<<<dim3(grid),dim3(threads)>>>(...)` launcher (to_cuda.py:245-247),
 * adding the stream and the error check the reference lacks. */
int frnn_launch(frnn_kernel_t k, const uint32_t grid[3], const uint32_t block[3],
                uint32_t lds_bytes, void* stream, const void* args, size_t arg_bytes);

/* Size of the library's static scratch buffer, per GPU (see frnn_launch_static). */
#define FRNN_STATIC_SCRATCH_BYTES (64ull << 20)

/* One hidden buffer of a launch that is to live in the library's static scratch buffer. */
typedef struct frnn_scratch_slot {
  uint64_t arg_offset;     /* byte offset, in the argument block, of the 8-byte pointer field to fill in  */
  uint64_t scratch_offset; /* where the region starts inside the scratch buffer; a multiple of 256         */
  uint64_t bytes;          /* size of the region; offset + bytes <= FRNN_STATIC_SCRATCH_BYTES              */
  uint64_t clear;          /* non-zero: the region is zero-filled on `stream` before the kernel runs       */
} frnn_scratch_slot;

/* frnn_launch for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose
 * `forward` / `backward` allocate the checkpoints and saved sums with torch on every call
 * (twopass.py:224-228, 349-356).  Same as frnn_launch, except that the pointer fields of `args`
 * named by `slots` are filled in by the library with addresses inside a buffer of
 * FRNN_STATIC_SCRATCH_BYTES that is part of the library's device image (every GPU the library runs on
 * holds one until the process ends).  The caller chooses the layout (`scratch_offset`), so several
 * launches can share regions: the forward kernel writes the checkpoints where the backward kernels
 * of the same call read them.  Inputs and outputs are still passed by the caller.  The call
 * allocates and frees nothing and never synchronises; regions marked `clear` are zeroed by a fill
 * kernel on `stream` (no memset node, so the call may be captured into a graph).  A region that does
 * not fit, is misaligned or overlaps another one of the same call is rejected with FRNN_ERR_ARG: use
 * frnn_launch with caller-allocated buffers for such sizes.  The buffer keeps what the last launch
 * left in it.  All calls on one GPU share it: calls whose kernels may overlap in time on one GPU
 * (other streams, other threads) race unless their regions are disjoint.  The buffer used is that of the
 * calling thread's current device, which must be the device `stream` belongs to (and the one the module was
 * loaded on).  The first call on each device looks the buffer's address up and must not be made during stream
 * capture.  The library must share the application's HIP runtime (see the head of this file): the call fails
 * with FRNN_ERR_NO_HIP when it finds itself bound to a second copy. */
int frnn_launch_static(frnn_kernel_t k, const uint32_t grid[3], const uint32_t block[3],
                       uint32_t lds_bytes, void* stream, const void* args, size_t arg_bytes,
                       const frnn_scratch_slot* slots, size_t nslots);

/* Unload a module.  Kernels obtained from it become invalid. */
int frnn_module_free(frnn_module_t m);

/* Number of compute units of the current device (for tile heuristics); <0 on failure. */
int frnn_device_cus(void);

#ifdef __cplusplus
}
#endif
#endif
