/* A host written in plain C, doing what the reference's own hosts do with a plugin
 * (crates/onnx-runtime-ep-nxrt-host/src/loader.rs:159-201 and the call sequence of
 * crates/onnx-runtime-ep-cuda/tests/matmul_nbits_gpu.rs:223-352): dlopen, negotiate, create the
 * factory and the provider, take its allocator, then build one MatMulNBits kernel through the kernel
 * mirror, run it at accuracy_level 0 and 4 on inputs made from integer formulas, and check the
 * result against a scalar loop in this file. A second part does the same with every tensor of the call
 * allocated through the nxmem allocator plugin the library also exports
 * (crates/onnx-runtime-memory-abi/include/nxmem_memory_abi.h:581-610, 698-718): negotiate, create the
 * factories, open the allocator of device 0, allocate, run, deallocate, and ask for the unload report;
 * it also checks the refusals (wrong mechanism, wrong device, unknown allocation, a capability that is
 * not offered) and that the provider, its kernels and its allocators may be released in any order.
 * Prints one line per step; exit status 0 = all good.
 *
 *   nxrt_roundtrip <path to libnxrt_ep_rocm.so>
 */
#include <dlfcn.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "nxmem_abi.h"
#include "nxrt_abi.h"
#include "nxrt_ep_rocm.h"

#define CHECK(cond, ...)                        \
  do {                                          \
    if (!(cond)) {                              \
      fprintf(stderr, "FAIL: " __VA_ARGS__);    \
      fprintf(stderr, "\n");                    \
      return 1;                                 \
    }                                           \
  } while (0)
#define OK(st, what) CHECK((st).code == 0, "%s: %s", what, (const char*)(st).message)

#define LOAD(name)                                        \
  name##_fn name##_p = (name##_fn)dlsym(lib, #name);      \
  CHECK(name##_p != NULL, "symbol %s missing", #name)

typedef NxrtStatus (*NxrtNegotiate_fn)(const NxrtNegotiateRequest*, NxrtNegotiateResponse*);
typedef NxrtStatus (*NxrtCreateEpFactories_fn)(NxrtEpFactoryVtable**, size_t, size_t*);
typedef NxrtRocmEp* (*nxrt_rocm_ep_from_vtable_fn)(const NxrtEpVtable*);
typedef NxrtStatus (*nxrt_rocm_matmul_nbits_create_fn)(NxrtRocmEp*, const NxrtRocmMatMulNBitsAttrs*, const NxrtTensorDesc*, uint32_t, NxrtRocmMatMulNBits**);
typedef void (*nxrt_rocm_matmul_nbits_set_constant_inputs_fn)(NxrtRocmMatMulNBits*, const uint8_t*, uint32_t);
typedef NxrtStatus (*nxrt_rocm_matmul_nbits_execute_fn)(NxrtRocmMatMulNBits*, const NxrtRocmTensorView*, uint32_t, NxrtRocmTensorView*, uint32_t, void*, uint64_t);
typedef const char* (*nxrt_rocm_matmul_nbits_last_variant_fn)(const NxrtRocmMatMulNBits*);
typedef void (*nxrt_rocm_matmul_nbits_release_fn)(NxrtRocmMatMulNBits*);
typedef uint64_t (*nxrt_rocm_live_provider_count_fn)(void);
typedef NxmemStatus (*NxmemNegotiate_fn)(const NxmemNegotiateRequest*, NxmemNegotiateResponse*);
typedef NxmemStatus (*NxmemCreateAllocatorFactories_fn)(const NxmemAllocatorFactoryVtable**, uint64_t, uint64_t*);
typedef NxmemStatus (*NxmemQueryUnloadReadiness_fn)(NxmemUnloadReport*);

enum { M = 3, N = 70, K = 320, BS = 32, KB = K / BS };

static NxrtRocmTensorView view(void* data, uint32_t dtype, uint32_t ndim, const uint64_t* shape)
{
  NxrtRocmTensorView v;
  memset(&v, 0, sizeof(v));
  v.data = data;
  v.dtype = dtype;
  v.ndim = ndim;
  v.shape = shape;
  v.device_type = NXRT_DEVICE_ROCM;
  v.device_index = 0;
  return v;
}

int main(int argc, char** argv)
{
  CHECK(argc == 2, "usage: nxrt_roundtrip <libnxrt_ep_rocm.so>");
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  CHECK(lib != NULL, "dlopen: %s", dlerror());
  LOAD(NxrtNegotiate);
  LOAD(NxrtCreateEpFactories);
  LOAD(nxrt_rocm_ep_from_vtable);
  LOAD(nxrt_rocm_matmul_nbits_create);
  LOAD(nxrt_rocm_matmul_nbits_set_constant_inputs);
  LOAD(nxrt_rocm_matmul_nbits_execute);
  LOAD(nxrt_rocm_matmul_nbits_last_variant);
  LOAD(nxrt_rocm_matmul_nbits_release);
  LOAD(nxrt_rocm_live_provider_count);
  LOAD(NxmemNegotiate);
  LOAD(NxmemCreateAllocatorFactories);
  LOAD(NxmemQueryUnloadReadiness);

  /* negotiate: host speaks 1.0 .. 1.x */
  NxrtNegotiateRequest req = {sizeof(req), {1, 1, 0}};
  NxrtNegotiateResponse resp;
  memset(&resp, 0, sizeof(resp));
  resp.struct_size = sizeof(resp);
  OK(NxrtNegotiate_p(&req, &resp), "NxrtNegotiate");
  CHECK(resp.agreed_major == 1 && (resp.capability_flags & NXRT_CAP_ALLOCATOR), "negotiated %u.%u caps %llx", resp.agreed_major, resp.agreed_minor,
        (unsigned long long)resp.capability_flags);
  printf("negotiated %u.%u\n", resp.agreed_major, resp.agreed_minor);

  NxrtEpFactoryVtable* factory = NULL;
  size_t n_factories = 0;
  OK(NxrtCreateEpFactories_p(&factory, 1, &n_factories), "NxrtCreateEpFactories");
  CHECK(n_factories == 1 && factory && factory->num_devices >= 1, "no factory or no device");
  printf("factory %s, %u device(s)\n", (const char*)factory->name, factory->num_devices);

  NxrtEpVtable* ep_vt = NULL;
  OK(factory->create_ep(factory->ctx, 0, &ep_vt), "create_ep");
  CHECK(ep_vt->device_type == NXRT_DEVICE_ROCM, "device_type %u", ep_vt->device_type);
  NxrtAllocatorVtable* alloc = NULL;
  OK(ep_vt->get_allocator(ep_vt->ctx, &alloc), "get_allocator");

  /* operands from integer formulas, as the reference's tests make theirs */
  static float a[M * K], scales[N * KB], bias[N], y[M * N], y4[M * N], want[M * N];
  static uint8_t b[N * KB * BS / 2], zp[N * ((KB + 1) / 2)];
  for (int i = 0; i < M * K; ++i) a[i] = (float)((i * 37 + 11) % 29 - 14) / 8.0f;
  for (int i = 0; i < N * KB; ++i) scales[i] = 0.005f + (float)((i * 13) % 17) / 2048.0f;
  for (int i = 0; i < N; ++i) bias[i] = (float)(i % 7) - 3.0f;
  for (size_t i = 0; i < sizeof(b); ++i) b[i] = (uint8_t)((i * 151 + 7) % 256);
  for (size_t i = 0; i < sizeof(zp); ++i) zp[i] = (uint8_t)((i * 89 + 3) % 256);
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double sum = 0.0;
      for (int k = 0; k < K; ++k) {
        const int blk = k / BS;
        const uint8_t byte = b[(n * KB + blk) * (BS / 2) + (k % BS) / 2];
        const int q = (k & 1) ? (byte >> 4) : (byte & 15);           /* low nibble = even k */
        const uint8_t zbyte = zp[n * ((KB + 1) / 2) + blk / 2];
        const int z = (blk & 1) ? (zbyte >> 4) : (zbyte & 15);
        sum += (double)a[m * K + k] * ((double)(q - z) * (double)scales[n * KB + blk]);
      }
      want[m * N + n] = (float)(sum + bias[n]);
    }

  struct { void** dev; const void* host; size_t bytes; } ups[5];
  void *da, *db, *ds, *dz, *dbias, *dy;
  ups[0].dev = &da; ups[0].host = a; ups[0].bytes = sizeof(a);
  ups[1].dev = &db; ups[1].host = b; ups[1].bytes = sizeof(b);
  ups[2].dev = &ds; ups[2].host = scales; ups[2].bytes = sizeof(scales);
  ups[3].dev = &dz; ups[3].host = zp; ups[3].bytes = sizeof(zp);
  ups[4].dev = &dbias; ups[4].host = bias; ups[4].bytes = sizeof(bias);
  for (int i = 0; i < 5; ++i) {
    *ups[i].dev = alloc->alloc(alloc->ctx, ups[i].bytes, 256);
    CHECK(*ups[i].dev != NULL, "allocator returned NULL");
    OK(alloc->copy_from_host(alloc->ctx, *ups[i].dev, (const uint8_t*)ups[i].host, ups[i].bytes), "copy_from_host");
  }
  dy = alloc->alloc(alloc->ctx, sizeof(y), 256);
  CHECK(dy != NULL, "allocator returned NULL");

  NxrtRocmEp* ep = nxrt_rocm_ep_from_vtable_p(ep_vt);
  CHECK(ep != NULL, "ep_from_vtable");
  const uint64_t sh_a[2] = {M, K}, sh_b[3] = {N, KB, BS / 2}, sh_s[2] = {N, KB}, sh_z[2] = {N, (KB + 1) / 2}, sh_bias[1] = {N}, sh_y[2] = {M, N};
  const uint8_t constant[6] = {0, 1, 1, 1, 1, 1};
  float* outs[2] = {y, y4};
  for (int pass = 0; pass < 2; ++pass) {
    NxrtRocmMatMulNBitsAttrs attrs;
    memset(&attrs, 0, sizeof(attrs));
    attrs.struct_size = sizeof(attrs);
    attrs.present = 0x1f;                     /* K, N, bits, block_size, accuracy_level */
    attrs.K = K;
    attrs.N = N;
    attrs.bits = 4;
    attrs.block_size = BS;
    attrs.accuracy_level = pass == 0 ? 0 : 4;
    NxrtRocmMatMulNBits* kernel = NULL;
    OK(nxrt_rocm_matmul_nbits_create_p(ep, &attrs, NULL, 0, &kernel), "matmul_nbits_create");
    nxrt_rocm_matmul_nbits_set_constant_inputs_p(kernel, constant, 6);
    NxrtRocmTensorView in[6];
    in[0] = view(da, NXRT_DT_FLOAT32, 2, sh_a);
    in[1] = view(db, NXRT_DT_UINT8, 3, sh_b);
    in[2] = view(ds, NXRT_DT_FLOAT32, 2, sh_s);
    in[3] = view(dz, NXRT_DT_UINT8, 2, sh_z);
    in[4] = view(NULL, NXRT_DT_INT32, 0, NULL);          /* g_idx absent */
    in[5] = view(dbias, NXRT_DT_FLOAT32, 1, sh_bias);
    NxrtRocmTensorView out = view(dy, NXRT_DT_FLOAT32, 2, sh_y);
    OK(nxrt_rocm_matmul_nbits_execute_p(kernel, in, 6, &out, 1, NULL, 0), "matmul_nbits_execute");
    OK(alloc->copy_to_host(alloc->ctx, (uint8_t*)outs[pass], dy, sizeof(y)), "copy_to_host");
    OK(alloc->sync(alloc->ctx), "sync");
    double num = 0.0, den = 0.0;
    for (int i = 0; i < M * N; ++i) {
      num += ((double)outs[pass][i] - want[i]) * ((double)outs[pass][i] - want[i]);
      den += (double)want[i] * want[i];
    }
    const double rel = sqrt(num / den);
    printf("accuracy_level %d: variant %s, rel-L2 %.3e\n", pass == 0 ? 0 : 4, nxrt_rocm_matmul_nbits_last_variant_p(kernel), rel);
    CHECK(rel <= (pass == 0 ? 1e-5 : 1e-2), "result off: %.3e", rel);     /* int8 activations cost a few 1e-3 (matmul_nbits.rs:10986) */
    nxrt_rocm_matmul_nbits_release_p(kernel);
  }

  void* frees[6] = {da, db, ds, dz, dbias, dy};
  for (int i = 0; i < 6; ++i) alloc->free(alloc->ctx, frees[i]);

  /* ---- the same call with every tensor allocated through the nxmem allocator plugin ---- */
  NxmemNegotiateRequest mreq;
  memset(&mreq, 0, sizeof(mreq));
  mreq.struct_size = sizeof(mreq);
  mreq.host_range.major_min = 1;
  mreq.host_range.major_max = 1;
  mreq.host_range.minor_min = 0;
  mreq.host_range.minor_max = NXMEM_ABI_VERSION_MINOR;
  mreq.host_capability_flags = NXMEM_CAP_ALLOCATOR | NXMEM_CAP_DEFERRED_RELEASE;
  NxmemNegotiateResponse mresp;
  memset(&mresp, 0, sizeof(mresp));
#define MOK(st, what) do { NxmemStatus s_ = (st); CHECK(s_.code == NXMEM_STATUS_OK, "%s: code %u %s", what, s_.code, (const char*)s_.message); } while (0)
#define MREFUSED(st, want, what) do { NxmemStatus s_ = (st); CHECK(s_.code == (want), "%s: expected status %d, got %u %s", what, (int)(want), s_.code, (const char*)s_.message); } while (0)
  MOK(NxmemNegotiate_p(&mreq, &mresp), "NxmemNegotiate");
  CHECK(mresp.agreed_major == 1 && mresp.capability_flags == NXMEM_CAP_ALLOCATOR, "nxmem negotiated %u.%u caps %llx", mresp.agreed_major, mresp.agreed_minor,
        (unsigned long long)mresp.capability_flags);
  const NxmemAllocatorFactoryVtable* mfactories[16];
  uint64_t n_mfactories = 0;
  MOK(NxmemCreateAllocatorFactories_p(mfactories, 16, &n_mfactories), "NxmemCreateAllocatorFactories");
  CHECK(n_mfactories >= 1 && mfactories[0]->device.tier == NXMEM_TIER_DEVICE && mfactories[0]->device.index == 0, "no nxmem factory for device 0");
  const NxmemAllocatorFactoryVtable* mf = mfactories[0];
  NxmemOpenRequest open_req;
  memset(&open_req, 0, sizeof(open_req));
  open_req.struct_size = sizeof(open_req);
  open_req.abi_minor = mresp.agreed_minor;
  open_req.device.tier = NXMEM_TIER_DEVICE;
  open_req.device.index = 0;
  open_req.required_capability_flags = NXMEM_CAP_ALLOCATOR;
  const NxmemAllocatorVtable* mal = NULL;
  NxmemOpenRequest bad_open = open_req;
  bad_open.required_capability_flags = NXMEM_CAP_ALLOCATOR | NXMEM_CAP_VIRTUAL_BACKING;
  MREFUSED(mf->open_allocator(mf->ctx, &bad_open, &mal), NXMEM_STATUS_UNSUPPORTED_CAPABILITY, "open_allocator with virtual backing required");
  bad_open = open_req;
  bad_open.device.index = 7;
  MREFUSED(mf->open_allocator(mf->ctx, &bad_open, &mal), NXMEM_STATUS_WRONG_DEVICE, "open_allocator for another device");
  MOK(mf->open_allocator(mf->ctx, &open_req, &mal), "open_allocator");
  CHECK(mal && mal->allocate && mal->deallocate && mal->retain && mal->release, "a required allocator slot is NULL");
  CHECK(!mal->virtual_backing && !mal->shared_mapping && !mal->enqueue_release && !mal->drain_releases && !mal->pending_release_count && !mal->release_allocation,
        "an optional slot that is not offered must be NULL");
  printf("nxmem allocator %s, mechanism %llx\n", (const char*)mal->name, (unsigned long long)mal->mechanism_id);

  const size_t sizes[6] = {sizeof(a), sizeof(b), sizeof(scales), sizeof(zp), sizeof(bias), sizeof(y)};
  const void* hosts[6] = {a, b, scales, zp, bias, NULL};
  NxmemAllocation held[6];
  for (int i = 0; i < 6; ++i) {
    NxmemAllocRequest ar;
    memset(&ar, 0, sizeof(ar));
    ar.struct_size = sizeof(ar);
    ar.mechanism_id = mal->mechanism_id;
    ar.allocation_id = 1000 + (uint64_t)i;
    ar.device = mal->device;
    ar.bytes = sizes[i];
    ar.align = 256;
    NxmemAllocResult res;
    memset(&res, 0, sizeof(res));
    if (i == 0) {
      NxmemAllocRequest wrong = ar;
      wrong.mechanism_id ^= 1;
      MREFUSED(mal->allocate(mal->ctx, &wrong, &res), NXMEM_STATUS_WRONG_MECHANISM, "allocate for another mechanism");
      wrong = ar;
      wrong.device.index = 5;
      MREFUSED(mal->allocate(mal->ctx, &wrong, &res), NXMEM_STATUS_WRONG_DEVICE, "allocate for another device");
      wrong = ar;
      wrong.struct_size = 8;
      MREFUSED(mal->allocate(mal->ctx, &wrong, &res), NXMEM_STATUS_SHORT_STRUCT, "allocate with a short request");
    }
    MOK(mal->allocate(mal->ctx, &ar, &res), "nxmem allocate");
    CHECK(res.ptr != NULL && res.owned_bytes >= sizes[i] && res.mapped_bytes >= sizes[i] && ((uintptr_t)res.ptr & 255) == 0, "nxmem allocate result");
    memset(&held[i], 0, sizeof(held[i]));
    held[i].struct_size = sizeof(held[i]);
    held[i].mechanism_id = ar.mechanism_id;
    held[i].allocation_id = ar.allocation_id;
    held[i].device = ar.device;
    held[i].ptr = res.ptr;
    held[i].bytes = sizes[i];
    held[i].align = 256;
    if (hosts[i]) OK(alloc->copy_from_host(alloc->ctx, res.ptr, (const uint8_t*)hosts[i], sizes[i]), "copy_from_host into nxmem memory");
  }
  NxmemUnloadReport report;
  MOK(NxmemQueryUnloadReadiness_p(&report), "NxmemQueryUnloadReadiness");
  CHECK(report.struct_size == sizeof(report) && report.live_allocators == 1 && report.live_allocations == 6, "unload report with the call's tensors live: %llu allocators, %llu allocations",
        (unsigned long long)report.live_allocators, (unsigned long long)report.live_allocations);
  {
    NxrtRocmMatMulNBitsAttrs attrs;
    memset(&attrs, 0, sizeof(attrs));
    attrs.struct_size = sizeof(attrs);
    attrs.present = 0x1f;
    attrs.K = K;
    attrs.N = N;
    attrs.bits = 4;
    attrs.block_size = BS;
    attrs.accuracy_level = 0;
    NxrtRocmMatMulNBits* kernel = NULL;
    OK(nxrt_rocm_matmul_nbits_create_p(ep, &attrs, NULL, 0, &kernel), "matmul_nbits_create (nxmem)");
    nxrt_rocm_matmul_nbits_set_constant_inputs_p(kernel, constant, 6);
    NxrtRocmTensorView in[6];
    in[0] = view(held[0].ptr, NXRT_DT_FLOAT32, 2, sh_a);
    in[1] = view(held[1].ptr, NXRT_DT_UINT8, 3, sh_b);
    in[2] = view(held[2].ptr, NXRT_DT_FLOAT32, 2, sh_s);
    in[3] = view(held[3].ptr, NXRT_DT_UINT8, 2, sh_z);
    in[4] = view(NULL, NXRT_DT_INT32, 0, NULL);
    in[5] = view(held[4].ptr, NXRT_DT_FLOAT32, 1, sh_bias);
    NxrtRocmTensorView out = view(held[5].ptr, NXRT_DT_FLOAT32, 2, sh_y);
    OK(nxrt_rocm_matmul_nbits_execute_p(kernel, in, 6, &out, 1, NULL, 0), "matmul_nbits_execute (nxmem)");
    static float ym[M * N];
    OK(alloc->copy_to_host(alloc->ctx, (uint8_t*)ym, held[5].ptr, sizeof(ym)), "copy_to_host from nxmem memory");
    OK(alloc->sync(alloc->ctx), "sync");
    CHECK(memcmp(ym, y, sizeof(ym)) == 0, "the call over nxmem-allocated tensors differs from the call over the provider's allocator");
    printf("nxmem-allocated tensors: variant %s, same bits as before\n", nxrt_rocm_matmul_nbits_last_variant_p(kernel));
    /* any order: the provider's vtable goes first, the kernel and the allocator handle keep the provider alive */
    ep_vt->release(ep_vt->ctx);
    CHECK(nxrt_rocm_live_provider_count_p() == 1, "the provider died while a kernel and an allocator still referred to it");
    nxrt_rocm_matmul_nbits_release_p(kernel);
    CHECK(nxrt_rocm_live_provider_count_p() == 1, "the provider died while an allocator still referred to it");
  }
  uint64_t unmapped = 0;
  {
    NxmemAllocation wrong = held[0];
    wrong.allocation_id = 4242;
    MREFUSED(mal->deallocate(mal->ctx, &wrong, &unmapped), NXMEM_STATUS_UNKNOWN_ALLOCATION, "deallocate of an unknown id");
    wrong = held[0];
    wrong.mechanism_id ^= 1;
    MREFUSED(mal->deallocate(mal->ctx, &wrong, &unmapped), NXMEM_STATUS_WRONG_MECHANISM, "deallocate for another mechanism");
    wrong = held[0];
    wrong.device.index = 3;
    MREFUSED(mal->deallocate(mal->ctx, &wrong, &unmapped), NXMEM_STATUS_WRONG_DEVICE, "deallocate for another device");
  }
  for (int i = 0; i < 6; ++i) {
    unmapped = 0;
    MOK(mal->deallocate(mal->ctx, &held[i], &unmapped), "nxmem deallocate");
    CHECK(unmapped == sizes[i], "deallocate reported %llu unmapped bytes of %llu", (unsigned long long)unmapped, (unsigned long long)sizes[i]);
  }
  MREFUSED(mal->deallocate(mal->ctx, &held[0], &unmapped), NXMEM_STATUS_UNKNOWN_ALLOCATION, "second deallocate of one allocation");
  mal->release(mal->ctx);
  mf->release(mf->ctx);
  MOK(NxmemQueryUnloadReadiness_p(&report), "NxmemQueryUnloadReadiness");
  CHECK(report.live_allocators == 0 && report.live_allocations == 0 && report.live_views == 0 && report.queued_releases == 0,
        "unload report after release: %llu allocators, %llu allocations", (unsigned long long)report.live_allocators, (unsigned long long)report.live_allocations);
  printf("nxmem unload report: nothing live\n");

  alloc->release(alloc->ctx);
  factory->release(factory->ctx);
  CHECK(nxrt_rocm_live_provider_count_p() == 0, "a provider outlived its release");
  printf("released; roundtrip ok\n");
  dlclose(lib);
  return 0;
}
