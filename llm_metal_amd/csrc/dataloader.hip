// Batches of token ids from a pre-tokenized int32 file (include/data_hip.h).  Host code only.
#include "../../include/data_hip.h"

#include <fcntl.h>
#include <stdio.h>
#include <stdlib.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

struct TokenLoader {
    const int32_t *ids;
    size_t n_tokens, map_size, pos;
    int batch, seq;
};

extern "C" {

TokenLoader *token_loader_open(const char *path, int batch_size, int seq_len)
{
    const int fd = open(path, O_RDONLY);
    if (fd < 0) { fprintf(stderr, "[DataLoader] Cannot open: %s\n", path); return nullptr; }
    struct stat st;
    void *p = MAP_FAILED;
    if (fstat(fd, &st) == 0 && st.st_size > 0) p = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (p == MAP_FAILED) { fprintf(stderr, "[DataLoader] mmap failed for: %s\n", path); return nullptr; }
    TokenLoader *dl = new TokenLoader{(const int32_t *)p, (size_t)st.st_size / sizeof(int32_t), (size_t)st.st_size, 0, batch_size, seq_len};
    printf("[DataLoader] Loaded %s: %zu tokens (pre-tokenized)\n", path, dl->n_tokens);
    return dl;
}

void token_loader_free(TokenLoader *dl)
{
    if (!dl) return;
    munmap((void *)dl->ids, dl->map_size);
    delete dl;
}

int token_loader_next(TokenLoader *dl, uint32_t *input, uint32_t *target)
{
    const size_t n = (size_t)dl->batch * (size_t)dl->seq;
    if (dl->pos + n + 1 > dl->n_tokens) { dl->pos = 0; return -1; }
    const int32_t *src = dl->ids + dl->pos;                // rows of a batch are consecutive stretches of the stream
    for (size_t i = 0; i < n; i++) { input[i] = (uint32_t)src[i]; target[i] = (uint32_t)src[i + 1]; }
    dl->pos += n;
    return 0;
}

void token_loader_reset(TokenLoader *dl) { dl->pos = 0; }

void token_loader_shuffle(TokenLoader *dl)
{
    const size_t max_offset = dl->n_tokens / 2;
    if (max_offset > 0) dl->pos = (size_t)(rand() % (int)max_offset);
}

size_t token_loader_n_batches(const TokenLoader *dl)
{
    const size_t n = (size_t)dl->batch * (size_t)dl->seq;
    return n && dl->n_tokens ? (dl->n_tokens - 1) / n : 0;
}

size_t token_loader_n_tokens(const TokenLoader *dl) { return dl->n_tokens; }
size_t token_loader_position(const TokenLoader *dl) { return dl->pos; }

}  // extern "C"
