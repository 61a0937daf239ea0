/* A host written in plain C, doing what the reference's own hosts do with a plugin
 * (crates/onnx-runtime-ep-nxrt-host/src/loader.rs:159-201 and the call sequence of
 * crates/onnx-runtime-ep-cuda/tests/matmul_nbits_gpu.rs:223-352): dlopen, negotiate, create the
 * factory and the provider, take its allocator, then build one MatMulNBits kernel through the kernel
 * mirror, run it at accuracy_level 0 and 4 on inputs made from integer formulas, and check the
 * result against a scalar loop in this file. Prints one line per step; exit status 0 = all good.
 *
 *   nxrt_roundtrip <path to libnxrt_ep_rocm.so>
 */
#include <dlfcn.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

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
  alloc->release(alloc->ctx);
  ep_vt->release(ep_vt->ctx);
  factory->release(factory->ctx);
  CHECK(nxrt_rocm_live_provider_count_p() == 0, "a provider outlived its release");
  printf("released; roundtrip ok\n");
  dlclose(lib);
  return 0;
}
