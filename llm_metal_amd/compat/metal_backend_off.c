/*
 * The 30 symbols of the reference's legacy backend (src/core/metal_backend.h:8-102) for a build without Metal.
 *
 * The kept model structs pull in tensor.c / layers.c / attention.c / lora.c / optimizer.c, which reference these
 * symbols but call only four of them once metal_is_initialized() answers 0: every dispatch sits behind that test
 * and the files then take their CPU branches.  This unit gives the answer and makes every other symbol a loud
 * stop, so a stray call cannot go unnoticed.  Compiled inside the reference tree:
 *
 *   cc -I<reference>/src -c metal_backend_off.c
 */
#include "core/metal_backend.h"
#include <stdio.h>
#include <stdlib.h>

int metal_init(const char *shader_path) { (void)shader_path; return -1; }
void metal_cleanup(void) {}
int metal_is_initialized(void) { return 0; }
void metal_synchronize(void) {}
void metal_free_buffer(void *buf) { (void)buf; }
void *metal_create_shared_buffer(size_t bytes) { (void)bytes; return NULL; }
void *metal_buffer_contents(void *buf) { (void)buf; return NULL; }

static void no_backend(const char *fn)
{
    fprintf(stderr, "%s: the legacy Metal backend is not part of this build (metal_is_initialized() is 0)\n", fn);
    abort();
}
#define OFF no_backend(__func__)

void metal_matmul(void *a, void *b, void *c, int M, int K, int N, int ta, int tb)
{ (void)a; (void)b; (void)c; (void)M; (void)K; (void)N; (void)ta; (void)tb; OFF; }
void metal_matmul_batched(void *a, void *b, void *c, int batch, int M, int K, int N, int ta, int tb)
{ (void)a; (void)b; (void)c; (void)batch; (void)M; (void)K; (void)N; (void)ta; (void)tb; OFF; }
void metal_layer_norm_residual(void *x, void *res, void *out, void *gamma, void *beta, int batch, int dim, float eps)
{ (void)x; (void)res; (void)out; (void)gamma; (void)beta; (void)batch; (void)dim; (void)eps; OFF; }
void metal_flash_attention(void *q, void *k, void *v, void *o, int B, int H, int N, int D, float scale, int causal)
{ (void)q; (void)k; (void)v; (void)o; (void)B; (void)H; (void)N; (void)D; (void)scale; (void)causal; OFF; }
void metal_flash_attention_backward(void *q, void *k, void *v, void *o, void *d_o, void *dq, void *dk, void *dv,
                                    int B, int H, int N, int D, float scale, int causal)
{ (void)q; (void)k; (void)v; (void)o; (void)d_o; (void)dq; (void)dk; (void)dv; (void)B; (void)H; (void)N; (void)D; (void)scale; (void)causal; OFF; }
void metal_layer_norm(void *x, void *out, void *gamma, void *beta, int batch, int dim, float eps)
{ (void)x; (void)out; (void)gamma; (void)beta; (void)batch; (void)dim; (void)eps; OFF; }
void metal_layer_norm_backward(void *x, void *dy, void *gamma, void *dx, void *dgamma, void *dbeta, int batch, int dim, float eps)
{ (void)x; (void)dy; (void)gamma; (void)dx; (void)dgamma; (void)dbeta; (void)batch; (void)dim; (void)eps; OFF; }
void metal_gelu(void *in, void *out, int n) { (void)in; (void)out; (void)n; OFF; }
void metal_gelu_backward(void *in, void *dy, void *dx, int n) { (void)in; (void)dy; (void)dx; (void)n; OFF; }
void metal_rope(void *x, void *out, int B, int H, int N, int D, int offset)
{ (void)x; (void)out; (void)B; (void)H; (void)N; (void)D; (void)offset; OFF; }
void metal_rope_backward(void *dy, void *dx, int B, int H, int N, int D, int offset)
{ (void)dy; (void)dx; (void)B; (void)H; (void)N; (void)D; (void)offset; OFF; }
void metal_embedding(void *table, void *idx, void *out, int vocab, int dim, int seq)
{ (void)table; (void)idx; (void)out; (void)vocab; (void)dim; (void)seq; OFF; }
void metal_embedding_backward(void *dy, void *idx, void *dtable, int vocab, int dim, int seq)
{ (void)dy; (void)idx; (void)dtable; (void)vocab; (void)dim; (void)seq; OFF; }
void metal_softmax_ce_loss(void *logits, void *targets, void *loss, void *dlogits, int batch, int vocab)
{ (void)logits; (void)targets; (void)loss; (void)dlogits; (void)batch; (void)vocab; OFF; }
void metal_adamw_update(void *p, void *g, void *m, void *v, int n, float lr, float b1, float b2, float eps, float wd, int step)
{ (void)p; (void)g; (void)m; (void)v; (void)n; (void)lr; (void)b1; (void)b2; (void)eps; (void)wd; (void)step; OFF; }
void metal_add(void *a, void *b, void *out, int n) { (void)a; (void)b; (void)out; (void)n; OFF; }
void metal_mul(void *a, void *b, void *out, int n) { (void)a; (void)b; (void)out; (void)n; OFF; }
void metal_rms_norm(void *x, void *out, void *gamma, int batch, int dim, float eps)
{ (void)x; (void)out; (void)gamma; (void)batch; (void)dim; (void)eps; OFF; }
void metal_rms_norm_backward(void *x, void *dy, void *gamma, void *dx, void *dgamma, int batch, int dim, float eps)
{ (void)x; (void)dy; (void)gamma; (void)dx; (void)dgamma; (void)batch; (void)dim; (void)eps; OFF; }
void metal_silu(void *in, void *out, int n) { (void)in; (void)out; (void)n; OFF; }
void metal_silu_backward(void *in, void *dy, void *dx, int n) { (void)in; (void)dy; (void)dx; (void)n; OFF; }
void metal_lora_forward(void *x, void *a, void *b, void *delta, int M, int in_f, int out_f, int rank)
{ (void)x; (void)a; (void)b; (void)delta; (void)M; (void)in_f; (void)out_f; (void)rank; OFF; }
void metal_dequantize_4bit(void *packed, void *scales, void *zeros, void *out, int n, int group)
{ (void)packed; (void)scales; (void)zeros; (void)out; (void)n; (void)group; OFF; }
