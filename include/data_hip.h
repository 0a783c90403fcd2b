/*
 * data_hip.h — the data step in front of sft_train_step: batches of token ids from a pre-tokenized file, as the
 * reference's run_sft feeds them (main.c:436-470 over src/data/dataloader.c:51-141).
 */
#ifndef DATA_HIP_H
#define DATA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct TokenLoader TokenLoader;

/* dataloader_create_from_tokens (src/data/dataloader.c:51-83): the file is an array of int32 token ids, mapped, not
 * copied.  NULL (message on stderr) when it cannot be opened or mapped. */
TokenLoader *token_loader_open(const char *path, int batch_size, int seq_len);
void token_loader_free(TokenLoader *dl);
/* dataloader_next_batch (src/data/dataloader.c:97-123), writing the ids straight into the uint32 arrays that
 * sft_train_step takes (the reference goes through float tensors and casts, main.c:446-453):
 * input[b*seq + s] = ids[pos + b*seq + s], target[...] = ids[pos + b*seq + s + 1]; advances pos by batch*seq.
 * Returns 0, or -1 at the end of an epoch (fewer than batch*seq + 1 ids left): pos is then reset to 0 and nothing is
 * written. */
int token_loader_next(TokenLoader *dl, uint32_t *input, uint32_t *target);
void token_loader_reset(TokenLoader *dl);                 /* src/data/dataloader.c:125-127 */
/* src/data/dataloader.c:129-135: pos = rand() % (n_tokens / 2) */
void token_loader_shuffle(TokenLoader *dl);
size_t token_loader_n_batches(const TokenLoader *dl);     /* (n_tokens - 1) / (batch*seq), src/data/dataloader.c:137-141 */
size_t token_loader_n_tokens(const TokenLoader *dl);
size_t token_loader_position(const TokenLoader *dl);

#ifdef __cplusplus
}
#endif
#endif /* DATA_HIP_H */
