#include <stdio.h>
#include <string.h>
#include <stddef.h>
extern "C" {
int g_extra_ok = 0; unsigned char g_args[8192]; size_t g_nargs = 0; unsigned g_dims[7]; void* g_stream; void* g_kparams;
int hipModuleLoadData(void** m, const void* image) { *m = (void*)0x1111; return 0; }
int hipModuleUnload(void* m) { return 0; }
int hipModuleGetFunction(void** f, void* m, const char* n) { *f = (void*)0x2222; return 0; }
int hipModuleLaunchKernel(void* f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz, unsigned sh, void* stream, void** kp, void** extra) {
  g_dims[0]=gx; g_dims[1]=gy; g_dims[2]=gz; g_dims[3]=bx; g_dims[4]=by; g_dims[5]=bz; g_dims[6]=sh; g_stream = stream; g_kparams = kp;
  g_extra_ok = extra && extra[0] == (void*)1 && extra[2] == (void*)2 && extra[4] == (void*)3;
  g_nargs = *(size_t*)extra[3]; memcpy(g_args, extra[1], g_nargs); return 0; }
const char* hipGetErrorString(int e) { return "fake"; }
int hipGetDevice(int* d) { *d = 0; return 0; }
int hipDeviceGetAttribute(int* v, int a, int d) { *v = 256; return 0; }
int hipGetLastError() { return 0; }
}
