/* qk_gguf.h -- read-only GGUF access for the hot path's callers: tensor directory, scalar and
 * string metadata, split shards, and the eight tensors of one MoE layer.
 *
 * Stands for the reference's reader (src/gguf.h:54-198: class Gguf, open / find / kvInt / kvStr)
 * and for its MoE tensor-set loader (src/main.cpp:1265-1311, loadMoeT).  Same file handling:
 * GGUF version 2 or 3, mmap of the whole file, data section aligned to general.alignment
 * (default 32), and a first shard "<prefix>-00001-of-000NN.gguf" pulls in its siblings named by
 * split.count.  Unlike the reference every offset and length read from the file is checked
 * against the mapping, and a malformed file is an error return, never an exit.
 *
 * Host-only: no GPU call is made; tensor data pointers point into the mapping and stay valid
 * until qkg_close.  Errors are reported through qkk_last_error() (include/qk_kernels.h).
 */
#ifndef QK_GGUF_H
#define QK_GGUF_H

#include <stdint.h>

#include "qk_kernels.h"

#ifdef __cplusplus
extern "C" {
#endif

#define QKG_EFORMAT (-6)   /* not a GGUF file, unsupported version, truncated or inconsistent */
#define QKG_ENOTFOUND (-7) /* no tensor / key of that name */
#define QKG_EIO (-8)       /* open / stat / mmap failed */

typedef struct qkg_file qkg_file;

/* reference src/gguf.h:48-52 (GgufTensor) plus what a caller needs to copy the tensor */
typedef struct qkg_tensor {
    const char *name;  /* NUL-terminated, owned by the file object */
    uint32_t type;     /* ggml type id (enum qkk_type for the ones the kernels read) */
    uint32_t n_dims;
    uint64_t ne[4];    /* ne[0] = row length; dimensions the file does not list are 1 */
    const void *data;  /* into the mapping of the shard that holds the tensor */
    uint64_t nbytes;   /* rows * row bytes for the types qkk_row_bytes() knows, else 0 */
    uint32_t shard;    /* 0-based index of that shard */
    uint32_t pad;
} qkg_tensor;

/* reference src/gguf.h:63-91 (Gguf::open).  NULL on failure. */
qkg_file *qkg_open(const char *path);
void qkg_close(qkg_file *f);

uint32_t qkg_version(const qkg_file *f);
uint32_t qkg_n_shards(const qkg_file *f);
uint64_t qkg_n_tensors(const qkg_file *f);
/* i-th tensor in name order (reference: iteration over Gguf::tensors(), src/gguf.h:98) */
int qkg_tensor_at(const qkg_file *f, uint64_t i, qkg_tensor *out);
/* reference src/gguf.h:93-96 (Gguf::find) */
int qkg_find(const qkg_file *f, const char *name, qkg_tensor *out);
/* Scalar integer / bool and string metadata of the first shard (reference src/gguf.h:103-110,
 * kvInt / kvStr; float and array values are skipped as there). */
int qkg_kv_int(const qkg_file *f, const char *key, uint64_t *out);
int qkg_kv_str(const qkg_file *f, const char *key, const char **out);

/* The tensors of MoE layer `layer` ("blk.<layer>.ffn_*"), checked as the reference checks them
 * (src/main.cpp:1265-1311): all eight present; router tensors F32; gate/up both IQ3_XXS; down
 * IQ4_XS or Q6_K; shared expert Q8_0; n_used = "<arch>.expert_used_count" (default 8) within
 * 1..16 and <= n_expert; plus what the reference leaves to the kernels: shapes consistent with
 * each other and every tensor's bytes inside the file. */
typedef struct qkg_moe_tensors {
    uint32_t n_embd, n_ff, n_expert, n_used;
    int32_t gu_type, down_type;
    qkg_tensor gate_inp, gate_inp_shexp, gate_exps, up_exps, down_exps, gate_shexp, up_shexp, down_shexp;
} qkg_moe_tensors;
int qkg_moe_layer(const qkg_file *f, uint32_t layer, qkg_moe_tensors *out);

#ifdef __cplusplus
}
#endif
#endif
