/*
 * C ABI of libios_runtime.so -- the MI355X (gfx950) execution engine of the inter-operator scheduler.
 *
 * The first four functions are drop-in replacements for the entry points of the reference runtime
 * (reference src/ios/ios_runtime.cu:1478-1519) that the reference Python glue binds with ctypes
 * (reference python/ios/contrib/ios_runtime.py:26-135).  Arguments have the same order and meaning.
 * Differences: they return int (0 = success, non-zero = failure, message via ios_last_error()) where the
 * reference returns void and terminates the process on errors; a caller that ignores the return value
 * sees the reference behaviour minus the exit().
 *
 * All pointers are owned by the caller and only used during the call.  Host buffers are float32,
 * C-contiguous, NCHW.  The library keeps process-wide state like the reference (one device
 * context, one stream pool); calls from several host threads are serialised by an internal lock, and
 * ios_last_error() reports the most recent failure of any thread.
 * JSON documents are the wire format exported by ios.Graph.export_config() / Block.export_config()
 * (reference python/ios/ir.py:855-865,1038-1046).
 */
#ifndef IOS_RUNTIME_H
#define IOS_RUNTIME_H

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Latency of a whole graph under its schedule.  Replaces graph_latency (src/ios/ios_runtime.cu:1480-1484).
 * results[repeat]: milliseconds per forward pass, each the mean of `number` individually timed passes.
 * stage_results[repeat * num_stages] (row-major, caller-zeroed): per-stage milliseconds, written only when
 * profile_stage_latency != 0; num_stages = total number of stages over all blocks.
 */
int graph_latency(const char *graph_json, int batch_size, int warmup, int number, int repeat,
                  int profile_stage_latency, float *results, float *stage_results);

/* Same for a single block document.  Replaces block_latency (src/ios/ios_runtime.cu:1486-1490). */
int block_latency(const char *block_json, int batch_size, int warmup, int number, int repeat,
                  int profile_stage_latency, float *results, float *stage_results);

/*
 * Latency of one candidate stage.  Replaces stage_latency (src/ios/ios_runtime.cu:1492-1498).
 * stage_json: [[operator config, ...] per group]; input_json: {producer name: [C, H, W]} for every
 * producer outside the stage.  profile_stage_latency must be 0.  results[repeat]: milliseconds per pass,
 * `number` passes issued back to back inside one timing bracket.
 */
int stage_latency(const char *stage_json, const char *input_json, int batch_size, int warmup, int number,
                  int repeat, int profile_stage_latency, float *results, float *stage_results);

/*
 * One inference.  Replaces graph_inference (src/ios/ios_runtime.cu:1500-1517).
 * input: batch_size x C x H x W; filter_data[i]: OC x IC/groups x KH x KW and bias_data[i]: OC for the
 * convolution named conv_names[i] (convolutions inside sequential operators included); unknown names are
 * reported on stdout and skipped, NULL data is an error.  output: batch_size x shape of the last operator;
 * the last stage of the schedule must have a single group.
 */
int graph_inference(const char *graph_json, int batch_size, float *input, int num_convs, char **conv_names,
                    float **filter_data, float **bias_data, float *output);

/* ---- extensions without a counterpart in the reference ------------------------------------------------ */

/*
 * graph_inference for callers that cannot allocate device memory (harnesses that forbid hipMalloc, tight serving
 * loops).  No counterpart in the reference.  Same arguments and results as graph_inference, but the call makes no
 * hipMalloc / hipFree and creates no events or streams (the library's per-device context - its streams and the address
 * of the static array - is created by the first call into the library that touches the device, whichever it is, and is
 * not part of this promise: call ios_device_info once beforehand where that matters): every device buffer of the pass (operator outputs, filters,
 * packed filters, split-K partial tiles and their ticket counters) is laid out in a static device array of
 * IOS_NO_ALLOC_SCRATCH_BYTES that device 0 holds from library load to process end.  A graph whose plan needs more
 * at the given batch size is refused with an error that names both figures.  Kernel configurations come from the
 * tuning cache where a shape was measured before and from the closed-form model otherwise (nothing is measured here);
 * operators run on one stream in schedule order.  All calls share the one array, which keeps the previous call's
 * contents (what must start at zero is cleared by a fill kernel); the library's lock serialises calls inside a
 * process, calls from several processes do not share the array.
 */
#define IOS_NO_ALLOC_SCRATCH_BYTES (256u << 20)
int graph_inference_no_alloc(const char *graph_json, int batch_size, float *input, int num_convs, char **conv_names,
                             float **filter_data, float **bias_data, float *output);

/* Numbering of the blocks of a split-K convolution whose K slices meet inside one XCD (host only, for tests): for a
 * launch over `tiles` output tiles and `split` K slices, writes for every block of the grid the tile it works on (-1:
 * the block has none and ends at once) and its slice, and returns the number of blocks; with null arrays or a capacity
 * below that number only the number is returned.  Blocks whose indices are equal modulo 8 run on one XCD, and all
 * slices of a tile have such indices. */
int ios_xcd_numbering(int tiles, int split, int *tile_of_block, int *slice_of_block, int capacity);

/* The three bfloat16 terms into which the "x3_*" convolution kernels split an fp32 operand, each as the upper half of a
 * 32-bit word (host only, for tests): terms[0] + terms[1] + terms[2], read as floats, equal x exactly for every normal x. */
void ios_split_bf16x3(float x, unsigned *terms);

/* Free device memory in bytes as hipMemGetInfo reports it (creates the device context if there is none yet), or -1. */
long long ios_device_free_bytes(void);

/* Message of the most recent failure (valid until the next failing call). */
const char *ios_last_error(void);

/* Options (set them before sessions are created):
 *   "executor" = "fused" (default: the groups of a stage share one kernel launch per level) | "fused_graph" (fused
 *       launches inside a hipGraph) | "streams" (one HIP stream per group, event fork/join) | "graph" (the stream form
 *       captured into a hipGraph and replayed).  The fused forms are the fast ones at small batches; at large ones
 *       (batch 64) the stream forms can be ahead by a little, because every convolution kernel configuration may serve a
 *       parallel stage there, also the few too heavy on registers or LDS to share any fused launch;
 *   "autotune" = "1" (default) | "0": measure convolution kernel configurations on first use, like the reference's
 *       cudnnFind-based selection (src/ios/ios_runtime.cu:150-205); "clear_tuning" = anything forgets them;
 *   "split_k_reduce" = "xcd" (default: the last block of a tile adds the split-K slices inside the convolution kernel,
 *       and the grid is numbered so that the slices of a tile run on one XCD and meet in its L2; used where a probe at
 *       start-up finds the dispatcher's round-robin placement, every block checks its own placement, and a mismatch
 *       makes the next synchronising call fail and switches the form off) | "inline" (the same with the slices anywhere
 *       on the device, exchanged through memory) | "kernel" (a second kernel adds them); same results bit for bit;
 *   "host_plan_split_k" = N: K slices of every matrix-path convolution in plans made without a device
 *       (ios_plan_describe, ios_plan_arena_bytes; 0 = the closed-form model's choice);
 *   "precision" = "fp32" | "bf16" | "fp16": reduced-precision modes of the matrix-path convolutions (bfloat16 or IEEE half
 *       operands, fp32 accumulation and outputs); "fp16" is the counterpart of the reference's USE_FLOAT16 build option
 *       (src/ios/ios_runtime.cu:19-43), with its range (operands beyond 65504 become infinite);
 *   "arena_reuse" = "1" (default) | "0": operator outputs, temporaries and split-K partial tiles whose lifetimes (first to
 *       last stage that touches them) do not intersect share device memory; the network input and the result never do.
 *       The reference allocates every output for the lifetime of the graph (src/ios/ios_runtime.cu:1273-1285, 1318-1327).
 *       With "0" every operator output survives the pass (ios_session_get_tensor on any node); needs no device;
 *   "commute_pool_conv" = "1" (default) | "0": an average pool that keeps the map size and the 1 x 1 convolution to no more
 *       channels that alone reads it change places: the convolution runs first without bias and activation, the pool
 *       then works on the convolution's channels and finishes with bias and activation (same result up to the order of
 *       fp32 roundings; the pool operator has no tensor of its own any more); needs no device;
 *   "thin_conv_min_pixels" = count (default 262144; negative: never): a 3 x 3 convolution of a 3-channel image with at least
 *       this many output pixels (batch x OH x OW) that has its stage to itself runs on a direct kernel bound by the bytes of
 *       its output instead of the matrix path (first layers at large batches); needs no device;
 *   "conv_variant" = index or -1 and "conv_split_k" = count or 0 force one convolution kernel configuration (testing). */
int ios_set_option(const char *key, const char *value);

/* JSON description of device 0 ({"name", "arch", "compute_units", ...}) into buf. */
int ios_device_info(char *buf, int cap);

/* JSON list of the convolution kernel configuration names this build holds, in index order, into buf; returns the
 * length (call again with a larger buffer when the return value >= cap).  Touches no device. */
int ios_conv_variant_names(char *buf, int cap);

/* Host-only planning: writes the JSON list of device operations for a graph into buf and returns its length
 * (call again with a larger buffer when the return value >= cap); -1 on error.  Touches no device. */
int ios_plan_describe(const char *graph_json, int batch_size, char *buf, int cap);

/* Host-only planning: bytes of device memory the plan of a graph lays out at a batch size (closed-form kernel
 * configurations); -1 on error.  Touches no device. */
long long ios_plan_arena_bytes(const char *graph_json, int batch_size);

/* Persistent session: plan once, keep weights and activations on the device, run many times. */
typedef struct ios_session ios_session;
ios_session *ios_session_create(const char *graph_json, int batch_size);   /* NULL on failure */
void ios_session_destroy(ios_session *session);
int ios_session_set_conv_weights(ios_session *session, int num_convs, char **conv_names, float **filter_data,
                                 float **bias_data);
int ios_session_set_input(ios_session *session, const float *input);
int ios_session_run(ios_session *session);                                  /* one forward pass, waits for it */
/* One forward pass queued behind the earlier ones without waiting, and the wait for everything queued: K passes
 * between two synchronisations run back to back on the device while the host's launch work overlaps the pass before.
 * That is a throughput figure.  The reference's timers do something else (src/ios/ios_runtime.cu:1419-1441: the device
 * is synchronised before every pass and every pass has its own pair of events): ios_session_measure follows them. */
int ios_session_enqueue(ios_session *session);
int ios_session_synchronize(ios_session *session);
int ios_session_get_output(ios_session *session, float *output);
/* Dense copy of an operator's output (batch x C x H x W) after a run.  Fails, with a message that says which, for an
 * operator whose output is never written as such (a ReLU applied by the convolution that reads it, a sum added by the
 * depth-wise convolution or the activation that reads it, the convolution and the addition of a residual unit whose result
 * the convolution's epilogue writes) and, under "arena_reuse" = "1", for one whose memory a later operator took over. */
int ios_session_get_tensor(ios_session *session, const char *node_name, float *output);
/* Same protocol and outputs as graph_latency, on the resident session. */
int ios_session_measure(ios_session *session, int warmup, int number, int repeat, int profile_stage_latency,
                        float *results, float *stage_results);
int ios_session_num_ops(ios_session *session);                              /* -1 on failure */
int ios_session_describe(ios_session *session, char *buf, int cap);         /* like ios_plan_describe */
/* ms[num_ops]: mean HIP-event time of each device operation launched `repeat` times back to back on one stream. */
int ios_session_profile_ops(ios_session *session, int warmup, int repeat, float *ms);

/* The kernel launches of one forward pass as the executor in force issues them (one per level of a multi-group stage
 * under the fused executors), in issue order, as a JSON array into buf: kernel name, stage, blocks, threads, the
 * operations behind it and their algorithmic flops and bytes.  Returns the length like ios_plan_describe. */
int ios_session_describe_launches(ios_session *session, char *buf, int cap);
/* ms[i] (capacity entries available): mean HIP-event time of launch i issued `repeat` times back to back on the launch stream. */
int ios_session_profile_launches(ios_session *session, int warmup, int repeat, float *ms, int capacity);

#ifdef __cplusplus
}
#endif

#endif /* IOS_RUNTIME_H */
