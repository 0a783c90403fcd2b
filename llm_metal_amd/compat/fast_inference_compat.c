/*
 * The reference-signature entry points of src/nn/fast_inference.h over the generation pipeline of the library
 * (fast_inference_compat.h, next to this file).  Compiled inside the reference tree in place of fast_inference.c:
 *
 *   cc -DFAST_METAL_H -I<reference>/src/nn -I<this repo>/include -c fast_inference_compat.c
 */
#include "fast_inference_compat.h"
#include "model_ref_compat.h"

static InferenceState *create(ModelDesc *m, int have, int max_seq_len, int use_fp16)
{
    InferenceState *s = NULL;
    if (have == 0) {
        const SFTModelRef ref = model_desc_ref(m, NULL);   /* adapters come later, through inference_state_set_lora */
        s = inference_state_create_from_ref(&ref, max_seq_len, use_fp16);
        model_desc_free(m);
    }
    return s;
}

InferenceState *inference_state_create(Qwen3Model *model, int max_seq_len, int use_fp16)
{
    ModelDesc m;
    return create(&m, model_desc_qwen3(&m, model), max_seq_len, use_fp16);
}

InferenceState *inference_state_create_gemma3(Gemma3Model *model, int max_seq_len, int use_fp16)
{
    ModelDesc m;
    return create(&m, model_desc_gemma3(&m, model), max_seq_len, use_fp16);
}

int qwen3_generate_fast(Qwen3Model *model, const uint32_t *prompt_tokens, int prompt_len, uint32_t *output_tokens,
                        int max_gen_len, int max_seq_len, int use_fp16)
{
    InferenceState *s = inference_state_create(model, max_seq_len, use_fp16);
    if (!s) return 0;
    const int n = inference_generate(s, prompt_tokens, prompt_len, output_tokens, max_gen_len);
    inference_state_free(s);
    return n;
}

int qwen3_generate_fast_batch(Qwen3Model *model, const uint32_t *prompt_tokens, int prompt_len, uint32_t *output_tokens,
                              int max_gen_len, int max_seq_len, int batch_size)
{
    /* the state's own single-sequence cache is not used by the batched pipeline: keep it as small as the call allows */
    (void)max_seq_len;
    InferenceState *s = inference_state_create(model, prompt_len + max_gen_len + 1, /* F16 */ 1);
    if (!s) return 0;
    const int n = inference_generate_batch(s, prompt_tokens, prompt_len, output_tokens, max_gen_len, batch_size);
    inference_state_free(s);
    return n;
}
