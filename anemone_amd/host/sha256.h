/* sha256.h -- SHA-256 over bytes given in pieces (sha256.c); private to the library's host sources. */
#ifndef ANEMONE_HOST_SHA256_H
#define ANEMONE_HOST_SHA256_H

#include <stdint.h>

#define SHA256_DIGEST_BYTES 32

struct sha256_stream {
    uint32_t state[8];
    uint64_t byte_count;
    unsigned char pending[64]; /* the bytes of a block not yet full */
};

void sha256_begin(struct sha256_stream *stream);
void sha256_feed(struct sha256_stream *stream, const void *bytes, uint64_t count);
void sha256_finish(struct sha256_stream *stream, unsigned char digest_out[SHA256_DIGEST_BYTES]);
void anemone_sha256(const void *bytes, uint64_t count, unsigned char digest_out[SHA256_DIGEST_BYTES]);

#endif
