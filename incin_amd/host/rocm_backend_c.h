/* Flat C view of incin_amd/host/rocm_backend.hpp, so that tests written in Python (ctypes) can drive the
 * C++ host mirror the way the reference's Rust tests drive its backends (tests/sdpa.rs).  Every call
 * returns an ErrorKind value (0 = success); the message of the last failure on the calling thread is kept
 * for incin_host_last_error().  Storages are opaque handles, released with incin_host_release(). */
#ifndef INCIN_ROCM_HOST_C_H
#define INCIN_ROCM_HOST_C_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct incin_host_storage incin_host_storage;

const char* incin_host_last_error(void);
int incin_host_from_bytes(const void* bytes, size_t nbytes, const int64_t* dims, int32_t rank, int32_t dtype, int32_t device,
                          incin_host_storage** out);
int incin_host_numel(const incin_host_storage* s, int64_t* out);
int incin_host_rank(const incin_host_storage* s, int32_t* out);
int incin_host_shape(const incin_host_storage* s, int64_t* dims_out);
int incin_host_strides(const incin_host_storage* s, int64_t* strides_out);      /* elements; 0 on a broadcast axis */
int incin_host_dtype(const incin_host_storage* s, int32_t* out);
int incin_host_to_bytes(const incin_host_storage* s, void* out, size_t capacity);
int incin_host_transpose(const incin_host_storage* s, int32_t a, int32_t b, incin_host_storage** out);
int incin_host_broadcast_as(const incin_host_storage* s, const int64_t* dims, int32_t rank, incin_host_storage** out);
int incin_host_narrow(const incin_host_storage* s, int32_t dim, int64_t start, int64_t len, incin_host_storage** out);
int incin_host_tag_causal(const incin_host_storage* mask, incin_host_storage** out);
int incin_host_tag_key_padding(const incin_host_storage* mask, const int32_t* lens, int64_t count, incin_host_storage** out);
/* *kind: 0 untagged (out is the mask as it was), 1 causal, 2 key padding, 3 both; reads the mask on the device and waits */
int incin_host_infer_mask_tag(const incin_host_storage* mask, int32_t* kind, incin_host_storage** out);
/* mask may be null; has_scale = 0 means Option::None (default 1/sqrt(D)) */
int incin_host_scaled_dot_product_attention(const incin_host_storage* q, const incin_host_storage* k, const incin_host_storage* v,
                                            const incin_host_storage* mask, int32_t has_scale, double scale,
                                            incin_host_storage** out);
/* the same forward and, for an upstream gradient of the output's shape, the gradients of q, k, v (fresh contiguous storages) */
int incin_host_attention_backward(const incin_host_storage* q, const incin_host_storage* k, const incin_host_storage* v,
                                  const incin_host_storage* mask, int32_t has_scale, double scale, const incin_host_storage* grad_out,
                                  incin_host_storage** out, incin_host_storage** dq, incin_host_storage** dk, incin_host_storage** dv);
void incin_host_release(incin_host_storage* s);
/* device address of the view's first element (for tests that rewrite an operand in place between replays of a recording) */
int incin_host_data_ptr(const incin_host_storage* s, void** out);
/* the stream the calling thread's operators launch on (NULL: the default stream) */
void incin_host_set_stream(void* stream);
/* recording of the calling thread's work on its stream into a launch graph; replays go to the calling thread's stream */
typedef struct incin_host_graph incin_host_graph;
int incin_host_begin_recording(int32_t device);
int incin_host_end_recording(incin_host_graph** out);
int incin_host_replay(const incin_host_graph* g);
void incin_host_release_graph(incin_host_graph* g);
/* pool counters of a device: allocations made on the device so far, buffers handed out from the pool, bytes idle in it */
int incin_host_pool_stats(int32_t device, int64_t* device_allocs, int64_t* reused, int64_t* idle_bytes);
int incin_host_trim_pool(int32_t device);
/* number of kernel launches (C-ABI sdpa calls) the last attention call on this thread made */
int64_t incin_host_last_launch_count(void);


/* ---- capability registry (rocm_capability.hpp).  Enumerations travel as their integer values, in the order the
 * header declares them.  device_kind: 0 cpu, 1 cuda, 2 wgpu, 3 metal, 4 rocm. ---- */
/* spelling of an enumeration value; what: 0 operation, 1 dtype, 2 layout, 3 math mode, 4 implementation, 5 device */
const char* incin_host_capability_name(int32_t what, int32_t value);
int32_t incin_host_capability_max_rank(void);
/* support level of a query: 0 native, 1 composed, 2 fallback, 3 unsupported.  For 3, *reason_kind gets the
 * UnsupportedReason variant (0 operation, 1 dtype, 2 layout, 3 rank, 4 training, 5 math mode) and `reason` its text. */
int incin_host_capability_support(int32_t device_kind, int32_t operation, int32_t dtype, int32_t layout, int32_t rank,
                                  int32_t training, int32_t math_mode, int32_t* reason_kind, char* reason, size_t capacity);
int32_t incin_host_capability_rule_count(int32_t device_kind);
/* one registration; dtypes / layouts / math_modes come back as bit masks over the enumeration values */
int incin_host_capability_rule(int32_t device_kind, int32_t index, int32_t* operation, uint32_t* dtypes, uint32_t* layouts,
                               int32_t* min_rank, int32_t* max_rank, int32_t* training, uint32_t* math_modes,
                               int32_t* implementation);
/* the generated tables for the rows this backend adds (summary over cpu and rocm, then both sections); returns the
 * length of the text, of which at most capacity - 1 bytes are written */
size_t incin_host_capability_docs(char* out, size_t capacity);


/* ---- validated descriptors and their executor (rocm_exec.hpp) ---- */
typedef struct incin_host_attention_spec incin_host_attention_spec;
/* the shape rule; kv_lens_count / q_lens_count < 0: no such counts; has_scale = 0: default 1/sqrt(D).  Needs no device. */
int incin_host_lower_attention(const int64_t* q_dims, int32_t q_rank, const int64_t* k_dims, int32_t k_rank, const int64_t* v_dims,
                               int32_t v_rank, int32_t dtype, int32_t causal, const int32_t* kv_lens, int64_t kv_lens_count,
                               int32_t has_scale, double scale, const int32_t* q_lens, int64_t q_lens_count,
                               incin_host_attention_spec** out);
int incin_host_attention_spec_out_dims(const incin_host_attention_spec* spec, int64_t* dims_out, int32_t* rank_out, int64_t* group_out);
int incin_host_execute_attention(const incin_host_attention_spec* spec, const incin_host_storage* const* inputs, int32_t n_inputs,
                                 incin_host_storage** out);
void incin_host_release_attention_spec(incin_host_attention_spec* spec);
int incin_host_reshape(const incin_host_storage* s, const int64_t* dims, int32_t rank, incin_host_storage** out);

/* ---- device detection (rocm_exec.hpp); kinds as for the capability registry ---- */
int32_t incin_host_is_compiled_in(int32_t kind);
int32_t incin_host_probe(int32_t kind);                    /* device ordinal, or -1 */
/* n < 0: the default preference order (cuda, rocm, metal, wgpu, cpu) */
int incin_host_detect_device(const int32_t* preference, int32_t n, int32_t* kind, int32_t* ordinal);

#ifdef __cplusplus
}
#endif
#endif
