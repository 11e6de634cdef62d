/*
 * The fixed device scratch of the entry point that allocates nothing (lng_static.hip owns the array,
 * lng_hip.cpp uses the address it hands out).
 *
 * Layout of the LNG_STATIC_SCRATCH_BYTES bytes, in order:
 *   partial outputs   LNG_STATIC_MAX_SLOTS x 64 f32   (row, kv head, chunk, query head of the group)
 *   partial (max,sum) LNG_STATIC_MAX_SLOTS x 2 f32
 */
#ifndef LNG_STATIC_H
#define LNG_STATIC_H

#include <stddef.h>

#include "../../include/lng_hip.h"

#define LNG_STATIC_MAX_SLOTS LNG_STATIC_SCRATCH_SLOTS /* the limit the C ABI states */
#define LNG_STATIC_O_BYTES ((size_t)LNG_STATIC_MAX_SLOTS * 64u * 4u)
#define LNG_STATIC_ML_BYTES ((size_t)LNG_STATIC_MAX_SLOTS * 2u * 4u)
#define LNG_STATIC_SCRATCH_BYTES (LNG_STATIC_O_BYTES + LNG_STATIC_ML_BYTES)
#define LNG_STATIC_MAX_DEVICES 64

#ifdef __cplusplus
extern "C" {
#endif
int lng_static_scratch_setup(int device);
void *lng_static_scratch(int device);
#ifdef __cplusplus
}
#endif
#endif /* LNG_STATIC_H */
