// KV-cache append: writes the new tokens' K and V rows into preallocated caches [B,Hkv,Smax,D] (or page pools
// [pages,Hkv,page_size,D] addressed through a block table) at per-batch positions.
// The reference grows K/V with op::concat on the sequence axis (reference src/Operation/OpTransform.cpp:306-357), which
// copies the whole history for every generated token; here only the new rows move.  HBM-bound by construction:
// 2 * B*Hkv*Lnew*D elements read and written once, 16 bytes per lane when rows allow it.

#include "sdpa_common.h"

namespace ttsdpa {

namespace {

template <int VEC>  // bytes per lane and access
__global__ __launch_bounds__(256) void kv_append_kernel(KvAppendArgs a) {
  const int row_bytes = a.D * a.esz;
  const int per_row = row_bytes / VEC;
  const long long rows = (long long)a.B * a.Hkv * a.Lnew;
  const long long total = rows * per_row;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += (long long)gridDim.x * 256) {
    const int piece = (int)(e % per_row);
    long long r = e / per_row;
    const int l = (int)(r % a.Lnew);
    r /= a.Lnew;
    const int hk = (int)(r % a.Hkv);
    const int b = (int)(r / a.Hkv);
    const int pos = (a.positions ? a.positions[b] : a.position) + l;
    if (pos < 0 || pos >= a.Smax) continue;  // no room: the row is dropped
    const char* ksrc = (const char*)a.kn + (b * a.kns[0] + hk * a.kns[1] + l * a.kns[2]) * a.esz + piece * VEC;
    const char* vsrc = (const char*)a.vn + (b * a.vns[0] + hk * a.vns[1] + l * a.vns[2]) * a.esz + piece * VEC;
    long long slab = b;  // contiguous cache: the batch entry; paged cache: the page that holds row pos
    int row = pos;
    if (a.block_table) {
      slab = a.block_table[(long long)b * a.bt_stride + (pos >> a.page_shift)];
      row = pos & ((1 << a.page_shift) - 1);
    }
    char* kdst = (char*)a.kc + (slab * a.kcs[0] + hk * a.kcs[1] + row * a.kcs[2]) * a.esz + piece * VEC;
    char* vdst = (char*)a.vc + (slab * a.vcs[0] + hk * a.vcs[1] + row * a.vcs[2]) * a.esz + piece * VEC;
    if (VEC == 16) {
      *(u32x4*)kdst = *(const u32x4*)ksrc;
      *(u32x4*)vdst = *(const u32x4*)vsrc;
    } else if (VEC == 4) {
      *(uint32_t*)kdst = *(const uint32_t*)ksrc;
      *(uint32_t*)vdst = *(const uint32_t*)vsrc;
    } else {
      *(uint16_t*)kdst = *(const uint16_t*)ksrc;
      *(uint16_t*)vdst = *(const uint16_t*)vsrc;
    }
  }
}

bool aligned_for(const KvAppendArgs& a, int vec) {
  auto ok = [&](const void* p, const long long* st) {
    if (((uintptr_t)p % vec) != 0) return false;
    for (int i = 0; i < 3; i++)
      if ((st[i] * a.esz) % vec != 0) return false;
    return true;
  };
  return (a.D * a.esz) % vec == 0 && ok(a.kc, a.kcs) && ok(a.vc, a.vcs) && ok(a.kn, a.kns) && ok(a.vn, a.vns);
}

}  // namespace

int launch_kv_append(const KvAppendArgs& a, hipStream_t stream) {
  const int vec = aligned_for(a, 16) ? 16 : aligned_for(a, 4) ? 4 : 2;
  const long long total = (long long)a.B * a.Hkv * a.Lnew * (a.D * a.esz / vec);
  long long nwg = (total + 255) / 256;
  if (nwg > 256 * 16) nwg = 256 * 16;
  if (nwg < 1) return 0;
  dim3 grid((unsigned)nwg), block(256);
  if (vec == 16) hipLaunchKernelGGL(kv_append_kernel<16>, grid, block, 0, stream, a);
  else if (vec == 4) hipLaunchKernelGGL(kv_append_kernel<4>, grid, block, 0, stream, a);
  else hipLaunchKernelGGL(kv_append_kernel<2>, grid, block, 0, stream, a);
  return (int)hipGetLastError();
}

}  // namespace ttsdpa
