/* The two symbols ONNX Runtime resolves when it loads this library as a plugin execution provider
 * (RegisterExecutionProviderLibrary): crates/onnx-runtime-ep-plugin/src/lib.rs:113-188 (the reference exports the same
 * pair from every EP shim through export_ep_factories!, e.g. crates/onnx-runtime-ep-cuda-plugin/src/lib.rs).
 *
 * The types are ONNX Runtime's (onnxruntime_c_api.h / onnxruntime_ep_c_api.h); where those headers are absent,
 * ort_plugin_ep_subset.h restates the part in use. */
#ifndef NXRT_ORT_PLUGIN_H_
#define NXRT_ORT_PLUGIN_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

struct OrtApiBase;
struct OrtLogger;
struct OrtEpFactory;
struct OrtStatus;

/* lib.rs:113-152 / factory.rs create_ep_factories: one factory ("RocmExecutionProvider", or `registration_name` when the
 * host gives one), written to factories[0]; *num_factories = 1. Errors come back as an OrtStatus of the host's making
 * (NULL = success): INVALID_ARGUMENT for a null output or max_factories == 0, NOT_IMPLEMENTED when the host has no plugin-EP
 * API. With no usable host API at all (null api_base, or a host older than the API version this library was built for)
 * there is nothing to make a status with: the call returns NULL and *num_factories stays 0.
 * The factory lists every AMD GPU among the host's hardware devices (GetSupportedDevices), creates one EP per GPU (CreateEp),
 * hands ORT a device allocator and a data transfer for that GPU's memory, and its EPs claim the com.microsoft::MatMulNBits
 * nodes the provider supports (per-slot dtype rule of crates/onnx-runtime-ep-cpu/src/kernels/mod.rs:197-209), one node per
 * fusion. No GPU is touched before the first allocation, copy or kernel. */
struct OrtStatus* CreateEpFactories(const char* registration_name, const struct OrtApiBase* api_base, const struct OrtLogger* default_logger,
                                    struct OrtEpFactory** factories, size_t max_factories, size_t* num_factories);

/* lib.rs:154-186 / factory.rs release_ep_factory: frees a factory CreateEpFactories returned. The host releases a factory's
 * EPs, allocators and data transfers first; if any is still alive the call answers with a FAIL status and the factory stays
 * valid. */
struct OrtStatus* ReleaseEpFactory(struct OrtEpFactory* factory);

#ifdef __cplusplus
}
#endif
#endif
