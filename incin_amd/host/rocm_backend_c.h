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
int incin_host_dtype(const incin_host_storage* s, int32_t* out);
int incin_host_to_bytes(const incin_host_storage* s, void* out, size_t capacity);
int incin_host_transpose(const incin_host_storage* s, int32_t a, int32_t b, incin_host_storage** out);
int incin_host_broadcast_as(const incin_host_storage* s, const int64_t* dims, int32_t rank, incin_host_storage** out);
int incin_host_narrow(const incin_host_storage* s, int32_t dim, int64_t start, int64_t len, incin_host_storage** out);
int incin_host_tag_causal(const incin_host_storage* mask, incin_host_storage** out);
int incin_host_tag_key_padding(const incin_host_storage* mask, const int32_t* lens, int64_t count, incin_host_storage** out);
/* mask may be null; has_scale = 0 means Option::None (default 1/sqrt(D)) */
int incin_host_scaled_dot_product_attention(const incin_host_storage* q, const incin_host_storage* k, const incin_host_storage* v,
                                            const incin_host_storage* mask, int32_t has_scale, double scale,
                                            incin_host_storage** out);
void incin_host_release(incin_host_storage* s);
/* number of kernel launches (C-ABI sdpa calls) the last attention call on this thread made */
int64_t incin_host_last_launch_count(void);

#ifdef __cplusplus
}
#endif
#endif
