/*
 * C ABI of the host-side network runtime (libdabnn_host.so): the surface of
 * bnn::Net (dabnn/net.h:50-61) as the reference's JNI wrapper exposes it
 * (dabnn/jni/JavaWrapper.cpp:17-89: readFile / readAsset / predict / getBlob /
 * dispose), for bindings that cannot call C++.
 *
 * Return value: 0 on success or a negative code; dabnet_last_error() holds the
 * message of the last failure on this thread.  The codes map the exception
 * types the reference throws: DABNET_ERUNTIME = std::runtime_error (BNN_ASSERT,
 * unsupported layer), DABNET_EINVALID = std::invalid_argument (unreadable
 * model file, dabnn/net.cpp:34-42), DABNET_EKEY = unknown blob name.
 */
#ifndef DABNN_NET_H
#define DABNN_NET_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define DABNET_API __attribute__((visibility("default")))
#else
#define DABNET_API
#endif

#define DABNET_OK 0
#define DABNET_ERUNTIME (-1)
#define DABNET_EINVALID (-2)
#define DABNET_EKEY (-3)

typedef struct dabnet dabnet_t;

DABNET_API const char *dabnet_last_error(void);

/* Net::create; NULL on failure. */
DABNET_API dabnet_t *dabnet_create(void);
/* dispose */
DABNET_API void dabnet_destroy(dabnet_t *net);

/* Images per run (the reference is fixed at 1, dabnn/net.cpp:64-65); call before reading the model. */
DABNET_API int dabnet_set_batch(dabnet_t *net, int batch);
/* The public flags of bnn::Net (dabnn/net.h:59-61); call before reading the model. */
DABNET_API int dabnet_set_flags(dabnet_t *net, int optimize, int run_fconv, int strict);
/* Replay the forward pass as one HIP graph from the third run on (default on). */
DABNET_API int dabnet_set_use_graph(dabnet_t *net, int on);
/* Per-layer-type timing, the reference's BNN_BENCHMARK build option (dabnn/layer.cpp:17-31). */
DABNET_API int dabnet_set_profile(dabnet_t *net, int on);
DABNET_API const char *dabnet_time_report(dabnet_t *net);

/* Net::read (dabnn/net.cpp:32-44) and Net::read_buf (:46); the buffer may be released after the call. */
DABNET_API int dabnet_read_file(dabnet_t *net, const char *path);
DABNET_API int dabnet_read_buf(dabnet_t *net, const void *buf, size_t len);

/*
 * No counterpart in the reference, which trusts the file: parses the model with every FlatBuffers offset checked against
 * len and runs the checks of Net::prepare (dabnn/net.cpp:56-270: version, shapes as common/Shaper.cpp, symmetric pads,
 * supported layer types, tensor sizes against layer geometry) on the host only -- no GPU is touched, nothing is built.
 * DABNET_OK, DABNET_EINVALID (truncated or corrupt buffer), DABNET_ERUNTIME (a BNN_ASSERT of the reference, or a tensor
 * that does not fit its layer) or DABNET_EKEY (a layer names a blob that does not exist).  dabnet_read_buf and
 * dabnet_read_file run the same checks before they allocate.
 */
DABNET_API int dabnet_check_model(const void *buf, size_t len, int run_fconv);

/* Net::run (dabnn/net.cpp:272-286): host_input holds batch x H x W x C floats (NHWC). Blocks until done. */
DABNET_API int dabnet_run(dabnet_t *net, const float *host_input);
/*
 * Same with the input already in device memory.  The layers read device_input where it lies (the reference's run wraps
 * its pointer without a copy), so it must stay valid and unchanged until the call returns; the net does not write to
 * it.  It is copied into the net's own input blob instead when it is not 256-byte aligned, when a layer rewrites the
 * input blob in place, or from the third time on that the address differs from the one the net's HIP graph was
 * captured with (a change of address costs a new capture).  NULL: the input blob already holds the input.
 */
DABNET_API int dabnet_run_device(dabnet_t *net, const float *device_input);

/* Name of the model's input blob (its shape through dabnet_blob_info). */
DABNET_API const char *dabnet_input_name(dabnet_t *net);

/* Net::get_blob (dabnn/net.cpp:288-290): shape as {n, h, w, c} (c in words for bit blobs), element type, bytes. */
DABNET_API int dabnet_blob_info(dabnet_t *net, const char *name, int shape[4], int *is_bit, size_t *bytes);
/* Copies the blob to host memory. */
DABNET_API int dabnet_get_blob(dabnet_t *net, const char *name, void *host_out, size_t bytes);

/* Layer list in execution order, for inspection (Layer::to_str). */
DABNET_API int dabnet_num_layers(dabnet_t *net);
DABNET_API const char *dabnet_layer_desc(dabnet_t *net, int index);

#ifdef __cplusplus
}
#endif

#endif /* DABNN_NET_H */
