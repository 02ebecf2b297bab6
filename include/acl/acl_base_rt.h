/*
 * Minimal stand-alone replacement for the vendor runtime header that
 * cann_ops_sparse.h includes (`#include <acl/acl_base_rt.h>`, reference
 * include/cann_ops_sparse.h:18).  Only the two things the CSR SpMV / SpMM
 * surface needs are defined here: the element-type enum and the stream type.
 *
 * Enumerator names are the ones the reference switches on
 * (sparse/common/aclsparse_descr.cpp:44-62); the numeric values follow the
 * publicly documented CANN `aclDataType` numbering so that integers passed by
 * existing callers keep their meaning.
 *
 * On this platform a stream is a HIP stream: `aclrtStream` is layout- and
 * value-compatible with `hipStream_t` (both are opaque pointers), so a caller
 * passes the `hipStream_t` it launches its own work on.
 */
#ifndef OPS_SPARSE_AMD_ACL_BASE_RT_H_
#define OPS_SPARSE_AMD_ACL_BASE_RT_H_

#include <stddef.h>
#include <stdint.h>

/* The enums of this ABI are passed by value and checked by the callee: a caller may hand over any int.  C++ leaves a
 * value outside an enum's enumerators undefined unless the enum has a fixed underlying type, so under C++ they get
 * one (int, what they are in C anyway: neither size nor calling convention changes). */
#ifndef OPSPARSE_ABI_ENUM
#ifdef __cplusplus
#define OPSPARSE_ABI_ENUM(name) enum name : int
#else
#define OPSPARSE_ABI_ENUM(name) enum name
#endif
#endif

#ifdef __cplusplus
extern "C" {
#endif

typedef OPSPARSE_ABI_ENUM(aclDataType) {
    ACL_DT_UNDEFINED = -1,
    ACL_FLOAT = 0,
    ACL_FLOAT16 = 1,
    ACL_INT8 = 2,
    ACL_INT32 = 3,
    ACL_UINT8 = 4,
    ACL_INT16 = 6,
    ACL_UINT16 = 7,
    ACL_UINT32 = 8,
    ACL_INT64 = 9,
    ACL_UINT64 = 10,
    ACL_DOUBLE = 11,
    ACL_BOOL = 12,
    ACL_STRING = 13,
    ACL_COMPLEX64 = 16,
    ACL_COMPLEX128 = 17,
    ACL_BF16 = 27,
    ACL_INT4 = 29,
    ACL_UINT1 = 30,
    ACL_COMPLEX32 = 33,
    ACL_HIFLOAT8 = 34,
    ACL_FLOAT8_E5M2 = 35,
    ACL_FLOAT8_E4M3FN = 36,
    ACL_FLOAT8_E8M0 = 37,
    ACL_FLOAT6_E3M2 = 38,
    ACL_FLOAT6_E2M3 = 39,
    ACL_FLOAT4_E2M1 = 40,
    ACL_FLOAT4_E1M2 = 41
} aclDataType;

/* A HIP stream handle (hipStream_t) passed through an opaque pointer. */
typedef void *aclrtStream;

#ifdef __cplusplus
}
#endif

#endif /* OPS_SPARSE_AMD_ACL_BASE_RT_H_ */
