/*
 * arcz_gguf.h -- GGUF (v2 / v3) model files for the matmul path: the file is memory-mapped, its metadata and tensor
 * directory parsed with every length checked against the file's size, and tensors are handed out as views of the
 * mapping.  Stands where the reference's GgufFile stands (src/gguf.h:93-361) for what the matmul path needs of it:
 * scalar and string metadata, the tensor directory, tensor bytes.  Split models, virtual tensors and array-valued
 * metadata beyond skipping them are not read.
 */
#ifndef ARCZ_GGUF_H
#define ARCZ_GGUF_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct arcz_gguf arcz_gguf;

/* GgufFile::GgufFile (src/gguf.h:108-131): maps and parses `path`.  NULL on failure (cannot open, not a GGUF file,
 * version < 2, counts or lengths the file cannot hold, an alignment that is no power of two, a tensor past the end of
 * the file, a type whose block size is unknown); arcz_gguf_error() says which.  Nothing stays mapped after a failure. */
arcz_gguf* arcz_gguf_open(const char* path);
void arcz_gguf_close(arcz_gguf* g);
const char* arcz_gguf_error(void);

uint32_t arcz_gguf_version(const arcz_gguf* g);
size_t arcz_gguf_n_kv(const arcz_gguf* g);
size_t arcz_gguf_n_tensors(const arcz_gguf* g);
uint64_t arcz_gguf_alignment(const arcz_gguf* g); /* "general.alignment", 32 when absent (src/gguf.h:344-346) */

/* Metadata (GgufFile::get_int / get_float / get_str, src/gguf.h:150-190): 1 and *out set when the key holds an integer
 * or bool (i64), an integer or a float but no bool (f64); 0 otherwise.  Strings: NULL when absent or not a string; valid until close. */
int arcz_gguf_kv_i64(const arcz_gguf* g, const char* key, int64_t* out);
int arcz_gguf_kv_f64(const arcz_gguf* g, const char* key, double* out);
const char* arcz_gguf_kv_str(const arcz_gguf* g, const char* key);

/* Tensor directory (GgufTensor, src/gguf.h:80-87): entry i; dims[0] is the contiguous dimension; data points into the
 * mapping and is valid until close.  0, or -1 for an index past the end.  Any out pointer may be NULL. */
int arcz_gguf_tensor(const arcz_gguf* g, size_t i, const char** name, uint32_t* type, uint32_t* ndim, uint64_t dims[8],
                     const void** data, uint64_t* nbytes);
/* GgufFile::find (src/gguf.h:133-136): index of the tensor called `name`, or -1. */
long arcz_gguf_find(const arcz_gguf* g, const char* name);
/* Elements per block and bytes per block of a ggml type (ggml_block_info, src/gguf.h:48-79); 0 for an unknown type. */
int arcz_ggml_block_info(uint32_t type, int* block_elems, int* block_bytes);

#ifdef __cplusplus
}
#endif
#endif
