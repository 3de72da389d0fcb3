/* C ABI over the host-side pipeline of this backend, for callers without a C++ toolchain (the Python tests and
 * bench.py bind it with ctypes). It wraps glasssix::excalibur::pipeline<Dtype>, whose C++ interface is the
 * reference's own (include/Excalibur/pipeline.hpp:17-47): construct from topology lines and a model file with a
 * device ordinal, forward() one NCHW input, read output blobs by name.
 * Failures inside the pipeline follow the reference's policy: a message on stderr and std::terminate(). */
#ifndef EXCALIBUR_CAPI_H_
#define EXCALIBUR_CAPI_H_
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct exc_pipeline exc_pipeline;

/* topology: the `.phai` text ('\n' separated); model_path: a `.racy` file or "" for dummy weights;
 * device: HIP ordinal (>= 0); dtype: 0 = pipeline<float>, 1 = pipeline<unsigned short> (fp16 storage). */
exc_pipeline* exc_pipeline_create(const char* topology, const char* model_path, int device, int dtype);
/* The reference's file-path constructors (include/Excalibur/pipeline.hpp:24-25, src/Excalibur/pipeline.cpp:580-587):
 * param_file is the path of a `.phai` file, model_file the path of a `.racy` file, or NULL / "" for dummy weights. */
exc_pipeline* exc_pipeline_create_from_files(const char* param_file, const char* model_file, int device, int dtype);
void exc_pipeline_destroy(exc_pipeline* p);
/* 1 (default): int8 convolution chains run as one fused plan, convolutions absorb the activation / sum layer behind
 * them; 0: every layer through forward_gpu, every blob stored. */
void exc_pipeline_set_fusion(exc_pipeline* p, int on);
int exc_pipeline_last_fused(exc_pipeline* p);
/* 1: a fused int8 plan replays its launches as one HIP graph from its second forward on; 0 (default; the replay
 * measured no faster than the calls on MI355X): one call per launch. */
void exc_pipeline_set_graphs(exc_pipeline* p, int on);
/* 1 if the last forward itself stored blob `name` as a float tensor; 0 for a blob a fused executor skipped, which
 * exc_pipeline_get then obtains by running the last input once more layer by layer. */
int exc_pipeline_blob_stored(exc_pipeline* p, const char* name);
/* Copies a host NCHW tensor into the pipeline's input blob and uploads it to the device. */
int exc_pipeline_set_input(exc_pipeline* p, const void* input, const int shape[4]);
/* pipeline::forward on the resident input; kernels are queued, not awaited. */
int exc_pipeline_run(exc_pipeline* p);
/* The same, but the results of the earlier forwards stay held, as a C++ caller may hold the blob_map of one forward
 * across the next: exc_pipeline_get_kept reads blob `name` of the forward `back` runs before the last one (1 = the one
 * before) like exc_pipeline_get. */
int exc_pipeline_run_keeping(exc_pipeline* p);
long exc_pipeline_get_kept(exc_pipeline* p, int back, const char* name, void* out, long capacity, int shape[4]);
int exc_pipeline_sync(exc_pipeline* p);
/* Stream slots (memory::set_stream_slot, pipeline::stream_slot; no counterpart in the reference): the calling thread works
 * in slot 0 unless it sets another (0..7); a pipeline created afterwards does all its device work on that slot's own HIP
 * stream, so exc_pipeline_run of pipelines made in different slots overlap on the GPU. exc_pipeline_sync and
 * exc_pipeline_get wait for the pipeline's own stream. Returns -1 for a slot outside the range. */
int exc_set_stream_slot(int slot);
int exc_pipeline_stream_slot(exc_pipeline* p);
/* set_input + run + sync */
int exc_pipeline_forward(exc_pipeline* p, const void* input, const int shape[4]);
/* Copies output blob or feature map `name` of the last forward to `out` if it fits in `capacity` elements;
 * returns its element count (-1 if unknown) and its shape. */
long exc_pipeline_get(exc_pipeline* p, const char* name, void* out, long capacity, int shape[4]);
/* Device time of part of a fused forward (no counterpart in the reference: a measurement aid). With
 * first_launch >= 0 every later fused forward records one event in front of its launch number first_launch
 * (0 = the input quantizer, or the stem when its kernel quantizes the input itself; -2 = the first convolution's launch,
 * whichever number it has) and one behind its last launch; -1 switches that off. exc_pipeline_last_span waits for
 * the device and returns the milliseconds between the two events of the last forward and, in *launches, how many
 * launches lay between them (0 and 0.0 if the last forward was not a fused one). The event pairs come from a ring of
 * 32: exc_pipeline_recent_spans waits for the device once and writes the spans of the latest forwards since
 * exc_pipeline_time_fused_span was called (oldest first, at most 32 and at most `capacity`), so that forwards queued
 * back to back are read without a synchronisation between them; it returns how many it wrote. */
void exc_pipeline_time_fused_span(exc_pipeline* p, int first_launch);
float exc_pipeline_last_span(exc_pipeline* p, int* launches);
int exc_pipeline_recent_spans(exc_pipeline* p, float* ms, int capacity);
/* Test and development switches, process-wide (nothing is read from the environment): "f16_nchw_only" = 1 keeps every
 * blob of pipeline<unsigned short> NCHW instead of NHWC between layers; any other name goes to exhip_set_option.
 * Returns 0, or an error code for an unknown name. */
int exc_set_option(const char* name, int value);
/* Newline-separated list of registered operator class names for a dtype (0 float, 1 unsigned short, 2 double).
 * Returns the length needed. */
size_t exc_registered_operations(int dtype, char* buf, size_t len);

#ifdef __cplusplus
}
#endif
#endif
