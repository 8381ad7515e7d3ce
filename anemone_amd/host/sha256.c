/* sha256.c -- SHA-256 as FIPS 180-4 defines it (sections 4.1.2, 4.2.2, 5.1.1, 5.3.3, 6.2), for the digests an EXL3
 * map's descriptor holds (source/exl3_descriptor.c:286-301 of the reference compares them as 64 hexadecimal digits; its
 * own source/sha256.h is the same function). A stream takes its bytes in any pieces. */
#include <string.h>

#include "sha256.h"

static const uint32_t round_constants[64] = {
    0x428a2f98u, 0x71374491u, 0xb5c0fbcfu, 0xe9b5dba5u, 0x3956c25bu, 0x59f111f1u, 0x923f82a4u, 0xab1c5ed5u, 0xd807aa98u, 0x12835b01u, 0x243185beu,
    0x550c7dc3u, 0x72be5d74u, 0x80deb1feu, 0x9bdc06a7u, 0xc19bf174u, 0xe49b69c1u, 0xefbe4786u, 0x0fc19dc6u, 0x240ca1ccu, 0x2de92c6fu, 0x4a7484aau,
    0x5cb0a9dcu, 0x76f988dau, 0x983e5152u, 0xa831c66du, 0xb00327c8u, 0xbf597fc7u, 0xc6e00bf3u, 0xd5a79147u, 0x06ca6351u, 0x14292967u, 0x27b70a85u,
    0x2e1b2138u, 0x4d2c6dfcu, 0x53380d13u, 0x650a7354u, 0x766a0abbu, 0x81c2c92eu, 0x92722c85u, 0xa2bfe8a1u, 0xa81a664bu, 0xc24b8b70u, 0xc76c51a3u,
    0xd192e819u, 0xd6990624u, 0xf40e3585u, 0x106aa070u, 0x19a4c116u, 0x1e376c08u, 0x2748774cu, 0x34b0bcb5u, 0x391c0cb3u, 0x4ed8aa4au, 0x5b9cca4fu,
    0x682e6ff3u, 0x748f82eeu, 0x78a5636fu, 0x84c87814u, 0x8cc70208u, 0x90befffau, 0xa4506cebu, 0xbef9a3f7u, 0xc67178f2u};

static uint32_t rotated(uint32_t word, unsigned right)
{
    return word >> right | word << (32u - right);
}

static void block_in(struct sha256_stream *stream, const unsigned char block[64])
{
    uint32_t schedule[64], v[8];
    for (unsigned t = 0; t < 16u; t++) {
        schedule[t] = (uint32_t)block[4u * t] << 24 | (uint32_t)block[4u * t + 1u] << 16 | (uint32_t)block[4u * t + 2u] << 8 | block[4u * t + 3u];
    }
    for (unsigned t = 16; t < 64u; t++) {
        const uint32_t near = schedule[t - 15u], far = schedule[t - 2u];
        schedule[t] = schedule[t - 16u] + (rotated(near, 7) ^ rotated(near, 18) ^ near >> 3) + schedule[t - 7u] +
                      (rotated(far, 17) ^ rotated(far, 19) ^ far >> 10);
    }
    memcpy(v, stream->state, sizeof v);
    for (unsigned t = 0; t < 64u; t++) {
        const uint32_t a = v[0], e = v[4];
        const uint32_t first = v[7] + (rotated(e, 6) ^ rotated(e, 11) ^ rotated(e, 25)) + ((e & v[5]) ^ (~e & v[6])) + round_constants[t] + schedule[t];
        const uint32_t second = (rotated(a, 2) ^ rotated(a, 13) ^ rotated(a, 22)) + ((a & v[1]) ^ (a & v[2]) ^ (v[1] & v[2]));
        memmove(v + 1, v, 7u * sizeof v[0]);
        v[4] += first;
        v[0] = first + second;
    }
    for (unsigned i = 0; i < 8u; i++) {
        stream->state[i] += v[i];
    }
}

void sha256_begin(struct sha256_stream *stream)
{
    static const uint32_t initial[8] = {0x6a09e667u, 0xbb67ae85u, 0x3c6ef372u, 0xa54ff53au, 0x510e527fu, 0x9b05688cu, 0x1f83d9abu, 0x5be0cd19u};
    memcpy(stream->state, initial, sizeof initial);
    stream->byte_count = 0;
}

void sha256_feed(struct sha256_stream *stream, const void *bytes, uint64_t count)
{
    const unsigned char *from = bytes;
    unsigned held = (unsigned)(stream->byte_count % 64u);
    stream->byte_count += count;
    if (held != 0u) { /* fill the block that is part full */
        const uint64_t room = 64u - held, taken = count < room ? count : room;
        memcpy(stream->pending + held, from, (size_t)taken);
        from += taken;
        count -= taken;
        if (held + taken < 64u) {
            return;
        }
        block_in(stream, stream->pending);
    }
    for (; count >= 64u; from += 64, count -= 64u) {
        block_in(stream, from);
    }
    memcpy(stream->pending, from, (size_t)count);
}

void sha256_finish(struct sha256_stream *stream, unsigned char digest_out[SHA256_DIGEST_BYTES])
{
    const uint64_t bit_count = stream->byte_count * 8u;
    unsigned char tail[72] = {0x80};
    /* a one bit, zeros to 56 bytes modulo 64, then the bit count, most significant byte first */
    const unsigned held = (unsigned)(stream->byte_count % 64u), zeros = (held < 56u ? 56u : 120u) - held;
    for (unsigned i = 0; i < 8u; i++) {
        tail[zeros + i] = (unsigned char)(bit_count >> (56u - 8u * i));
    }
    sha256_feed(stream, tail, zeros + 8u);
    for (unsigned i = 0; i < 8u; i++) {
        for (unsigned b = 0; b < 4u; b++) {
            digest_out[4u * i + b] = (unsigned char)(stream->state[i] >> (24u - 8u * b));
        }
    }
}

void anemone_sha256(const void *bytes, uint64_t count, unsigned char digest_out[SHA256_DIGEST_BYTES])
{
    struct sha256_stream stream;
    sha256_begin(&stream);
    sha256_feed(&stream, bytes, count);
    sha256_finish(&stream, digest_out);
}
