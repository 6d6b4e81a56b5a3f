// Error reporting, version query and the output un-permutation of the C ABI.
#include "pbs_common.h"
#include "../../include/pbs_hip.h"   // the definitions below are checked against the public declarations
#include <stdarg.h>
#include <stdio.h>

namespace {
thread_local char g_err[512] = "";
}

extern "C" const char* pbs_last_error(void) { return g_err; }

void pbs_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int pbs_arg_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return -1;
}

int pbs_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    pbs_set_error("%s: %s", what, hipGetErrorString(e));
    return (int)e;
  }
  return 0;
}

int pbs_require_no_static_lds(const void* kernel, const char* what) {
  hipFuncAttributes fa;
  const hipError_t e = hipFuncGetAttributes(&fa, kernel);
  if (e != hipSuccess) {
    pbs_set_error("%s: hipFuncGetAttributes: %s", what, hipGetErrorString(e));
    return (int)e;
  }
  if (fa.sharedSizeBytes != 0)
    return pbs_arg_error("%s: kernel built with %zu bytes of static LDS; its absolute LDS offsets assume none", what,
                         (size_t)fa.sharedSizeBytes);
  return 0;
}

extern "C" int pbs_abi_version(void) { return 1; }

namespace {

// out[b, h, q_idx[b, h, i], :] = in[b, h, i, :]; rows are 256 B, 16 lanes x 16 B each.
__global__ __launch_bounds__(256) void unpermute_kernel(const uint16_t* in, const int32_t* q_idx, uint16_t* out, int S,
                                                        int64_t rows_total, int64_t o_sb, int64_t o_sh, int64_t o_ss,
                                                        int H) {
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (row >= rows_total) return;
  const int c = threadIdx.x & 15;
  const int64_t bh = row / S;
  const int i = (int)(row % S);
  const int dst = q_idx ? q_idx[row] : i;
  const u32x4 v = *reinterpret_cast<const u32x4*>(in + row * 128 + c * 8);
  uint16_t* o = out + (bh / H) * o_sb + (bh % H) * o_sh + (int64_t)dst * o_ss + c * 8;
  *reinterpret_cast<u32x4*>(o) = v;
}

}  // namespace

extern "C" int pbs_unpermute(const void* o_perm, const int32_t* q_idx, void* o, int B, int H, int S, int head_dim,
                             int64_t o_sb, int64_t o_sh, int64_t o_ss, void* stream) {
  PBS_REQUIRE(o_perm && o, "pbs_unpermute: null tensor pointer");
  PBS_REQUIRE(head_dim == 128, "pbs_unpermute: head_dim must be 128, got %d", head_dim);
  PBS_REQUIRE(B > 0 && H > 0 && S > 0, "pbs_unpermute: empty shape");
  PBS_REQUIRE(o_sb % 8 == 0 && o_sh % 8 == 0 && o_ss % 8 == 0, "pbs_unpermute: strides must keep rows 16-byte aligned");
  // identity fast path: queries are not permuted and the output already sits in place
  if (!q_idx && o_perm == o) return 0;
  const int64_t rows = (int64_t)B * H * S;
  hipLaunchKernelGGL(unpermute_kernel, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)o_perm, q_idx, (uint16_t*)o, S, rows, o_sb, o_sh, o_ss, H);
  return pbs_check_launch("pbs_unpermute");
}
