/* C facade of the C++ host side's checkpoint loader (libferrite_host.so), for bindings that cannot call C++:
 * plain pointers and sizes, errors as a non-zero return with the message copied into `err`.
 *
 * The loader stands where the reference's Rust loader does (crates/ferrite-models/src/dsv41/weights.rs:814-905
 * SafetensorsIndex / TensorView; tensor names :333-354 and crates/ferrite-model/src/weights.rs:133-149); it is
 * host code above the kernel library, not part of the kernel library's ABI. */
#ifndef FERRITE_HOST_H
#define FERRITE_HOST_H

#include <stddef.h>
#include <stdint.h>

#include "../../include/ferrite_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define FERRITE_NAMING_DSV41 0 /* <prefix>.experts.<e>.w1|w2|w3.{weight,scale}, I8 + F8_E8M0 */
#define FERRITE_NAMING_GLM 1   /* <prefix>.experts.<e>.{gate,up,down}_proj.weight, BF16 / F32, quantised on load */

typedef struct ferrite_ckpt ferrite_ckpt; /* an opened shard: header index + read-only mapping */

ferrite_ckpt* ferrite_ckpt_open(const char* path, char* err, size_t errlen);
/* A checkpoint split over several files: further shards of the same checkpoint.  A tensor is taken from the first
 * shard that names it; ferrite_ckpt_data_start() is that of the first shard. */
int ferrite_ckpt_add_shard(ferrite_ckpt* ck, const char* path, char* err, size_t errlen);
void ferrite_ckpt_close(ferrite_ckpt* ck);
int64_t ferrite_ckpt_num_tensors(const ferrite_ckpt* ck);
uint64_t ferrite_ckpt_data_start(const ferrite_ckpt* ck);
/* 0 = found: dtype (NUL-terminated, <= 15 chars), shape (up to 8 dims), byte range in the data section. */
int ferrite_ckpt_tensor(const ferrite_ckpt* ck, const char* name, char dtype[16], int64_t shape[8], int* ndim,
                        uint64_t* begin, uint64_t* end);
/* Number of missing or wrongly shaped tensors of one layer's MoE; their names, one a line, go into `report`. */
int ferrite_ckpt_validate_moe(const ferrite_ckpt* ck, int naming, const char* prefix, const ferrite_moe_shape* shape,
                              char* report, size_t report_len);
/* Streams the layer into packed_dev (ferrite_moe_packed_bytes(shape) bytes) and router_bias_dev ([E] f32).
 * stats: [0] source bytes read, [1] packed bytes, [2] seconds, [3] workers used. */
int ferrite_ckpt_load_moe_layer(const ferrite_ckpt* ck, const char* hip_so_path, int device, int naming,
                                const char* prefix, const ferrite_moe_shape* shape, void* packed_dev,
                                void* router_bias_dev, int workers, int pad_scale_rows, double stats[4], char* err,
                                size_t errlen);

#ifdef __cplusplus
}
#endif
#endif
