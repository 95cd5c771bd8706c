/*
 * Binary range coder and symbol coders of the host side.
 *
 * The range coder produces and consumes exactly the byte stream of the
 * reference's arith.c (32-bit low/range, 15-bit probabilities, renormalise
 * while range < 0xff01, pending-0xff carry propagation), restated for
 * in-memory buffers.  tests/test_coder.py checks bit-compatibility against
 * the reference sources compiled in place.
 */
#include <math.h>
#include <string.h>
#include "../../include/nncp_host.h"

#define RC_MIN_BITS 16                       /* arith.c:36 */
#define RC_RANGE_MIN ((0xffu << 8) + 1)      /* arith.c:37 */
#define RC_RANGE_MAX (0xffu << RC_MIN_BITS)  /* arith.c:38 */
#define PROB_ONE (1 << NNCP_PROB_BITS)

static void emit(NNCPPutBit *s, int v)
{
    if (s->idx >= s->buf_size && s->sink && s->buf_size > 0) {
        s->sink(s->sink_opaque, s->buf, s->idx);
        s->n_flushed += s->idx;
        s->idx = 0;
    }
    if (s->idx < s->buf_size)
        s->buf[s->idx] = (uint8_t)v;
    else
        s->overflow = 1;
    s->idx++;
}

/* v in [0, 0x1fe].  Pending output is current_byte followed by (n_bytes - 1)
   bytes 0xff; a carry (v >= 0x100) ripples through them (arith.c:69-95). */
static void shift_out(NNCPPutBit *s, unsigned v)
{
    if (v == 0xff) {
        s->n_bytes++;
        return;
    }
    if (s->n_bytes > 0) {
        unsigned carry = v >> 8;
        emit(s, s->current_byte + carry);
        for (; s->n_bytes > 1; s->n_bytes--)
            emit(s, (0xff + carry) & 0xff);
    }
    s->n_bytes = 1;
    s->current_byte = (uint8_t)v;
}

static void renorm_enc(NNCPPutBit *s)
{
    while (s->range < RC_RANGE_MIN) { /* arith.c:113-118 */
        shift_out(s, s->low >> RC_MIN_BITS);
        s->low = (s->low & 0xffffu) << 8;
        s->range <<= 8;
    }
}

void nncp_put_bit_init(NNCPPutBit *s, uint8_t *buf, size_t buf_size)
{
    memset(s, 0, sizeof(*s));
    s->range = RC_RANGE_MAX;
    s->current_byte = 0xff;
    s->buf = buf;
    s->buf_size = buf_size;
}

void nncp_put_bit_set_sink(NNCPPutBit *s, void (*sink)(void *, const uint8_t *, size_t), void *opaque)
{
    s->sink = sink;
    s->sink_opaque = opaque;
}

void nncp_put_bit(NNCPPutBit *s, int prob0, int bit)
{
    uint32_t r0 = (uint32_t)(((uint64_t)s->range * (uint32_t)prob0) >> NNCP_PROB_BITS);
    if (bit) {
        s->low += r0;
        s->range -= r0;
    } else {
        s->range = r0;
    }
    renorm_enc(s);
}

size_t nncp_put_bit_flush(NNCPPutBit *s)
{
    int n = 0;
    uint32_t val, mask;
    if (s->range < (1u << RC_MIN_BITS)) { /* arith.c:169-173 */
        shift_out(s, s->low >> RC_MIN_BITS);
        s->low = (s->low & 0xffffu) << 8;
        s->range <<= 8;
    }
    while ((1u << (n + 1)) <= s->range) /* largest n with 2^n <= range */
        n++;
    val = s->low;
    mask = (1u << n) - 1;
    if (val & mask)
        val = (val + (1u << n)) & ~mask;
    shift_out(s, val >> RC_MIN_BITS);
    if (s->n_bytes > 0)
        shift_out(s, 0);
    if (s->sink) {
        s->sink(s->sink_opaque, s->buf, s->idx);
        s->n_flushed += s->idx;
        s->idx = 0;
    }
    return s->n_flushed + s->idx;
}

static void refill(NNCPGetBit *s) /* arith.c:209-231, zero padding past the end */
{
    s->range <<= 8;
    s->low <<= 8;
    if (s->idx < s->buf_len)
        s->low += s->buf[s->idx];
    s->idx++;
}

void nncp_get_bit_init(NNCPGetBit *s, const uint8_t *buf, size_t len)
{
    memset(s, 0, sizeof(*s));
    s->buf = buf;
    s->buf_len = len;
    for (int i = 0; i <= RC_MIN_BITS; i += 8)
        refill(s);
    s->range = RC_RANGE_MAX;
}

int nncp_get_bit(NNCPGetBit *s, int prob0)
{
    uint32_t r0 = (uint32_t)(((uint64_t)s->range * (uint32_t)prob0) >> NNCP_PROB_BITS);
    int b = s->low >= r0;
    if (b) {
        s->low -= r0;
        s->range -= r0;
    } else {
        s->range = r0;
    }
    while (s->range < RC_RANGE_MIN)
        refill(s);
    return b;
}

/* ---- symbol coders ------------------------------------------------------------ */

static int clamp_prob(long v)
{
    return v < 1 ? 1 : (v > PROB_ONE - 1 ? PROB_ONE - 1 : (int)v);
}

/* One binary decision per level of a balanced tree over [0, n_symb): the
   probability of the lower half is its float mass over the mass of the
   current range (cp_utils.c:299-323). */
void nncp_write_sym(NNCPPutBit *pb, const float *prob, int n_symb, int sym)
{
    int start = 0, n = n_symb;
    float p = 1.0f;
    while (n > 1) {
        int n0 = n >> 1;
        float p0 = vec_sum_f32(prob + start, n0);
        int prob0 = clamp_prob(lrintf(p0 * PROB_ONE / p));
        int bit = sym >= start + n0;
        nncp_put_bit(pb, prob0, bit);
        if (bit) { start += n0; n -= n0; p -= p0; }
        else { n = n0; p = p0; }
    }
}

int nncp_read_sym(NNCPGetBit *gb, const float *prob, int n_symb) /* cp_utils.c:325-349 */
{
    int start = 0, n = n_symb;
    float p = 1.0f;
    while (n > 1) {
        int n0 = n >> 1;
        float p0 = vec_sum_f32(prob + start, n0);
        int prob0 = clamp_prob(lrintf(p0 * PROB_ONE / p));
        if (nncp_get_bit(gb, prob0)) { start += n0; n -= n0; p -= p0; }
        else { n = n0; p = p0; }
    }
    return start;
}

/* The same tree walked on integer cumulative counts: no float work, O(log n)
   per symbol.  Every frequency is >= 1, so hi - lo >= n > 0. */
void nncp_write_sym_cdf(NNCPPutBit *pb, const uint16_t *cdf, int n_symb, int sym)
{
    int start = 0, n = n_symb;
    uint32_t lo = 0, hi = 65536;
    while (n > 1) {
        int n0 = n >> 1;
        uint32_t mid = cdf[start + n0];
        int prob0 = clamp_prob((long)(((uint64_t)(mid - lo) << NNCP_PROB_BITS) / (hi - lo)));
        int bit = sym >= start + n0;
        nncp_put_bit(pb, prob0, bit);
        if (bit) { start += n0; n -= n0; lo = mid; }
        else { n = n0; hi = mid; }
    }
}

/* nncp_write_sym_cdf from the entries it would read, in the order it reads them (nc_cdf_path) */
void nncp_write_sym_cdf_path(NNCPPutBit *pb, const uint16_t *path, int n_symb, int sym)
{
    int start = 0, n = n_symb;
    uint32_t lo = 0, hi = 65536;
    while (n > 1) {
        int n0 = n >> 1;
        uint32_t mid = *path++;
        int prob0 = clamp_prob((long)(((uint64_t)(mid - lo) << NNCP_PROB_BITS) / (hi - lo)));
        int bit = sym >= start + n0;
        nncp_put_bit(pb, prob0, bit);
        if (bit) { start += n0; n -= n0; lo = mid; }
        else { n = n0; hi = mid; }
    }
}

int nncp_read_sym_cdf(NNCPGetBit *gb, const uint16_t *cdf, int n_symb)
{
    int start = 0, n = n_symb;
    uint32_t lo = 0, hi = 65536;
    while (n > 1) {
        int n0 = n >> 1;
        uint32_t mid = cdf[start + n0];
        int prob0 = clamp_prob((long)(((uint64_t)(mid - lo) << NNCP_PROB_BITS) / (hi - lo)));
        if (nncp_get_bit(gb, prob0)) { start += n0; n -= n0; lo = mid; }
        else { n = n0; hi = mid; }
    }
    return start;
}

/* cp_utils.c:380-410 */
const void *nncp_bound_libnc(void)
{
    return (const void *)&nc_context_init;
}

float nncp_interp(const NNCPInterp *p, int64_t pos)
{
    for (int i = 0; i < p->n_steps; i++) {
        if (pos < p->pos[i]) {
            int64_t pos0 = i ? p->pos[i - 1] : 0;
            float t = (float)(pos - pos0) / (float)(p->pos[i] - pos0);
            return p->val[i] + t * (p->val[i + 1] - p->val[i]);
        }
    }
    if (p->decay_power == 0.0f || p->n_steps == 0)
        return p->val[p->n_steps];
    if (p->decay_power == 0.5f)
        return p->val[p->n_steps] / sqrtf((float)pos / (float)p->pos[p->n_steps - 1]);
    return p->val[p->n_steps] * pow((float)pos / (float)p->pos[p->n_steps - 1], -p->decay_power);
}
