/*
 * loader_hip.h — checkpoint files to weights: HuggingFace safetensors (F32 / F16 / BF16, one file or a directory of
 * shards) and GGUF v2 / v3 (F32 / F16 / Q8_0), the two formats the reference reads (src/data/safetensors.h,
 * src/data/gguf.h), and the tensor-name maps of its model loaders (src/nn/qwen3.c:211-371, src/nn/gemma3.c:176-285).
 *
 * Two routes from a file to a model:
 *   model_ref_load           fp32 host arrays in an SFTModelRef, as the reference's loaders fill their model structs
 *                            (4 bytes per weight of host memory); feeds sft_state_create_from_ref.
 *   inference_state_create_from_file (inference_hip.h)
 *                            tensor bytes go from the mapped file to HBM as they are and are converted there: F16 and
 *                            Q8_0 tensors are used bit for bit as stored (no dequantise -> requantise round trip).
 * The file functions need no GPU; model_file_load_wmat and the inference route do.
 */
#ifndef LOADER_HIP_H
#define LOADER_HIP_H

#include "sft_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ModelFile ModelFile;

/* element types; the values of F32 / F16 / Q8_0 are GGML's (src/data/gguf.h:8-10) */
enum { MF_F32 = 0, MF_F16 = 1, MF_Q8_0 = 8, MF_BF16 = 30 };

/* safetensors_open (src/data/safetensors.c:186-313) and gguf_open (src/data/gguf.c:97-186) in one: `path` is a
 * .safetensors file, a directory holding *.safetensors shards (read in alphabetical order), or a GGUF file (told by
 * its magic).  NULL, with a message on stderr, when the path cannot be read or parsed. */
ModelFile *model_file_open(const char *path);
void model_file_close(ModelFile *f);
int  model_file_is_gguf(ModelFile *f);
int  model_file_count(ModelFile *f);
const char *model_file_name(ModelFile *f, int i);
/* safetensors_find / gguf_find_tensor: 1 and the tensor's type, rank and shape when present, else 0.  The shape is as
 * stored: safetensors outermost first ([rows, cols]), GGUF innermost first ([cols, rows]). */
int  model_file_find(ModelFile *f, const char *name, int *dtype, int *ndim, uint64_t shape[4]);
/* rows and columns of a 1-D or 2-D tensor whatever the file's convention; 0 when absent or of higher rank */
int  model_file_matrix_shape(ModelFile *f, const char *name, int *rows, int *cols);
/* the tensor's bytes inside the mapped file (valid until model_file_close) */
const void *model_file_data(ModelFile *f, const char *name, size_t *nbytes);
/* safetensors_load_f32 (src/data/safetensors.c:343-384) / gguf_load_tensor_f32 (src/data/gguf.c:255-296): a malloc'd
 * fp32 copy (the caller frees it); F16 and BF16 widen exactly, Q8_0 is float(code) * float(scale). */
float *model_file_load_f32(ModelFile *f, const char *name, size_t *n_elements);
/* The tensor as a weight container in HBM: F16 (use_fp16 != 0) or Q8_0.  A tensor already in the wanted format is
 * uploaded as it is; anything else is converted on the GPU with the rounding of wmat_create_f16 / wmat_create_q8
 * (src/nn/wmat.c:19-75) applied to the widened values. */
WMat *model_file_load_wmat(ModelFile *f, const char *name, int use_fp16);

/* qwen3_load_safetensors / qwen3_load_gguf (src/nn/qwen3.c:211-371) and gemma3_load_safetensors
 * (src/nn/gemma3.c:176-285) up to the point where the model struct is filled: every tensor as fp32, the LM head tied to
 * the embedding when the file has none, Gemma3's norm weights + 1.0 (its RMSNorm is (1 + w) * norm(x)).  Shapes
 * come from the tensors themselves (the reference hard-codes its 4B / 1B configurations); RoPE bases are the
 * reference's (Qwen3 1e6; Gemma3 1e6 on layers with L % 6 == 0, else 1e4).  NULL if a tensor is missing or
 * mis-shaped.  Free with model_ref_free. */
SFTModelRef *model_ref_load(const char *path, ModelType model_type);
void model_ref_free(SFTModelRef *m);

#ifdef __cplusplus
}
#endif
#endif /* LOADER_HIP_H */
