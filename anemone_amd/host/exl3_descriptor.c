/*
 * exl3_descriptor.c -- an EXL3 map's descriptor against the open pack's records and the model (anemone_descriptor.h).
 * The rules, their order and their statuses are those of source/exl3_descriptor.c:706-1039 of the reference (the
 * contract is its header's, exl3_descriptor.h:7-40); the structure is this library's: the sidecar is read into a tree
 * once (json_tree.c), the rules are a walk over nodes, and the pack is a view of tensor records searched by name.
 */
#include <errno.h>
#include <fcntl.h>
#include <inttypes.h>
#include <limits.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include "anemone_descriptor.h"
#include "anemone_ops.h"
#include "json_tree.h"
#include "prepare_common.h"
#include "sha256.h"

#define DESCRIPTOR_FORMAT_VERSION 1u
#define WIDTH_KINDS 17u /* counts by bits_x2: K1 (2) to K8 (16); place 0 counts the layers of more than one width */
#define MIXED 0u
#define WIDTH_NAME_BYTES 16
#define NARROWEST 2u
#define SHOWN_BYTES 200
#define HASH_PIECE_BYTES 1048576u
#define SPACE_BYTES " \t\n\v\f\r"

struct check {
    const char *sidecar;
    const struct json_tree *tree;
    result_status status; /* of the first rule that failed */
};

/* one line naming the sidecar; the first failure's status stays. Always false, so a rule reads `holds || fail(...)` */
static bool fail(struct check *check, result_status status, const char *format, ...) __attribute__((format(printf, 3, 4)));
static bool fail(struct check *check, result_status status, const char *format, ...)
{
    char words[1024];
    va_list values;
    va_start(values, format);
    (void)vsnprintf(words, sizeof words, format, values);
    va_end(values);
    (void)fprintf(stderr, "anemone: exl3 descriptor %s: %s\n", check->sidecar, words);
    if (check->status == STATUS_OK) {
        check->status = status;
    }
    return false;
}

/* a value as the file writes it, for a line: its first bytes */
struct shown {
    int count;
    const char *bytes;
};

static struct shown shown_value(const struct check *check, uint32_t node)
{
    if (node == JSON_TREE_NONE) {
        return (struct shown){7, "nothing"};
    }
    const struct json_tree_node *n = &check->tree->nodes[node];
    const uint32_t count = n->end - n->begin;
    return (struct shown){(int)(count < SHOWN_BYTES ? count : SHOWN_BYTES), check->tree->text + n->begin};
}

static struct shown shown_key(const struct check *check, uint32_t node)
{
    const struct json_tree_node *n = &check->tree->nodes[node];
    const uint32_t count = n->key_end - n->key_begin;
    return (struct shown){(int)(count < SHOWN_BYTES ? count : SHOWN_BYTES), check->tree->text + n->key_begin};
}

static bool is_kind(const struct check *check, uint32_t node, enum json_tree_kind kind)
{
    return node != JSON_TREE_NONE && check->tree->nodes[node].kind == (uint32_t)kind;
}

/* decimal digits as Python writes an int that is not negative: no sign, no leading zero */
static bool decimal(const char *bytes, uint32_t count, uint64_t *number_out)
{
    uint64_t number = 0;
    if (count == 0 || (bytes[0] == '0' && count > 1u)) {
        return false;
    }
    for (uint32_t i = 0; i < count; i++) {
        const unsigned digit = (unsigned)bytes[i] - '0';
        if (digit > 9u || number > (UINT64_MAX - digit) / 10u) {
            return false;
        }
        number = number * 10u + digit;
    }
    *number_out = number;
    return true;
}

static bool whole_number(struct check *check, uint32_t node, const char *field, uint64_t *number_out)
{
    const struct json_tree_node *n = node != JSON_TREE_NONE ? &check->tree->nodes[node] : NULL;
    if (n != NULL && n->kind == JSON_TREE_NUMBER && decimal(check->tree->text + n->begin, n->end - n->begin, number_out)) {
        return true;
    }
    const struct shown s = shown_value(check, node);
    return fail(check, STATUS_INVALID_ARGUMENT, "%s: %.*s is no whole number", field, s.count, s.bytes);
}

static bool whole_number_is(struct check *check, uint32_t node, const char *field, uint64_t wanted, const char *whose)
{
    uint64_t number = 0;
    return whole_number(check, node, field, &number) &&
           (number == wanted || fail(check, STATUS_INVALID_ARGUMENT, "%s: %" PRIu64 ", but %s is %" PRIu64, field, number, whose, wanted));
}

/* a string with a byte other than a space in it and no NUL */
static bool is_text(struct check *check, uint32_t node, const char *field, const char **bytes_out, uint32_t *count_out)
{
    if (is_kind(check, node, JSON_TREE_STRING)) {
        const struct json_tree_node *n = &check->tree->nodes[node];
        const char *bytes = check->tree->strings + n->text_at;
        uint32_t spaces = 0;
        while (spaces < n->text_count && bytes[spaces] != '\0' && strchr(SPACE_BYTES, bytes[spaces]) != NULL) {
            spaces++;
        }
        if (spaces < n->text_count && memchr(bytes, '\0', n->text_count) == NULL) {
            *bytes_out = bytes;
            *count_out = n->text_count;
            return true;
        }
    }
    const struct shown s = shown_value(check, node);
    return fail(check, STATUS_INVALID_ARGUMENT, "%s: %.*s is no text", field, s.count, s.bytes);
}

static void hexadecimal(const unsigned char digest[SHA256_DIGEST_BYTES], char text_out[2 * SHA256_DIGEST_BYTES + 1])
{
    for (unsigned i = 0; i < SHA256_DIGEST_BYTES; i++) {
        (void)snprintf(text_out + 2u * i, 3, "%02x", digest[i]);
    }
}

/* a SHA-256 as the converter writes it, 64 lower-case hexadecimal digits, against a digest */
static bool digest_is(struct check *check, uint32_t node, const char *field, const unsigned char digest[SHA256_DIGEST_BYTES], const char *whose)
{
    char text[2 * SHA256_DIGEST_BYTES + 1];
    hexadecimal(digest, text);
    if (json_tree_string_is(check->tree, node, text)) {
        return true;
    }
    const struct shown s = shown_value(check, node);
    return fail(check, STATUS_INVALID_ARGUMENT, "%s: %.*s, but %s SHA-256 is %s", field, s.count, s.bytes, whose, text);
}

/* an object of exactly the named members (a key twice was refused before): found_out[i] the member named names[i] */
static bool members_exactly(struct check *check, uint32_t object, const char *owner, const char *const *names, uint32_t name_count,
                            uint32_t *found_out)
{
    if (!is_kind(check, object, JSON_TREE_OBJECT)) {
        const struct shown s = shown_value(check, object);
        return fail(check, STATUS_INVALID_ARGUMENT, "%s: %.*s is no object", owner, s.count, s.bytes);
    }
    for (uint32_t i = 0; i < name_count; i++) {
        found_out[i] = JSON_TREE_NONE;
    }
    for (uint32_t member = check->tree->nodes[object].child; member != JSON_TREE_NONE; member = check->tree->nodes[member].next) {
        uint32_t i = 0;
        while (i < name_count && !json_tree_key_is(check->tree, member, names[i])) {
            i++;
        }
        if (i == name_count) {
            const struct shown s = shown_key(check, member);
            return fail(check, STATUS_INVALID_ARGUMENT, "%s: a member %.*s, which the format does not define there", owner, s.count, s.bytes);
        }
        found_out[i] = member;
    }
    for (uint32_t i = 0; i < name_count; i++) {
        if (found_out[i] == JSON_TREE_NONE) {
            return fail(check, STATUS_INVALID_ARGUMENT, "%s: the member %s is missing", owner, names[i]);
        }
    }
    return true;
}

/* the converter's name of a width: K<whole>, K<whole>.5 for a half */
static void width_name(uint32_t bits_x2, char name_out[WIDTH_NAME_BYTES])
{
    if (bits_x2 == MIXED) {
        (void)snprintf(name_out, WIDTH_NAME_BYTES, "mixed");
    } else {
        (void)snprintf(name_out, WIDTH_NAME_BYTES, "K%u%s", bits_x2 / 2u, bits_x2 % 2u != 0 ? ".5" : "");
    }
}

/* {width: count}, every count at least 1, into counts by bits_x2 ("mixed" at MIXED: only a summary's layers may hold
 * it, and the comparison with what was counted refuses it elsewhere) */
static bool width_counts(struct check *check, uint32_t object, const char *field, uint64_t counts[WIDTH_KINDS])
{
    if (!is_kind(check, object, JSON_TREE_OBJECT)) {
        const struct shown s = shown_value(check, object);
        return fail(check, STATUS_INVALID_ARGUMENT, "%s: %.*s is no object", field, s.count, s.bytes);
    }
    for (uint32_t member = check->tree->nodes[object].child; member != JSON_TREE_NONE; member = check->tree->nodes[member].next) {
        uint32_t place = 0;
        char name[WIDTH_NAME_BYTES], counted[160];
        for (; place < WIDTH_KINDS; place++) {
            width_name(place, name);
            if (place != 1u && json_tree_key_is(check->tree, member, name)) {
                break;
            }
        }
        if (place == WIDTH_KINDS) {
            const struct shown s = shown_key(check, member);
            return fail(check, STATUS_INVALID_ARGUMENT, "%s: %.*s is no EXL3 width (K1 to K8, halves between)", field, s.count, s.bytes);
        }
        (void)snprintf(counted, sizeof counted, "%s.%s", field, name);
        if (!whole_number(check, member, counted, &counts[place])) {
            return false;
        }
        if (counts[place] == 0) {
            return fail(check, STATUS_INVALID_ARGUMENT, "%s: a count of 0 (a width that is not there is left out)", counted);
        }
    }
    return true;
}

static bool counts_agree(struct check *check, const char *field, const uint64_t given[WIDTH_KINDS], const uint64_t wanted[WIDTH_KINDS],
                         const char *whose)
{
    for (uint32_t place = 0; place < WIDTH_KINDS; place++) {
        if (given[place] != wanted[place]) {
            char name[WIDTH_NAME_BYTES];
            width_name(place, name);
            return fail(check, STATUS_INVALID_ARGUMENT, "%s: %" PRIu64 " of %s, but %s %" PRIu64, field, given[place], name, whose, wanted[place]);
        }
    }
    return true;
}

/* ---- the pack's records ---- */

/* names as unsigned bytes, a shorter one before a longer one it begins (include/anemone/pack.h:17-18) */
static int name_order(const char *left, uint32_t left_count, const char *right, uint32_t right_count)
{
    const uint32_t shared = left_count < right_count ? left_count : right_count;
    const int order = shared != 0 ? memcmp(left, right, shared) : 0;
    return order != 0 ? order : left_count < right_count ? -1 : left_count > right_count ? 1 : 0;
}

static bool view_is_sound(const struct exl3_pack_view *pack)
{
    if ((pack->tensors == NULL && pack->tensor_count != 0) || (pack->name_bytes == NULL && pack->name_byte_count != 0)) {
        return false;
    }
    for (uint32_t i = 0; i < pack->tensor_count; i++) {
        const struct pack_tensor *t = &pack->tensors[i];
        if (t->name_byte_count == 0 || t->name_byte_offset > pack->name_byte_count || t->name_byte_count > pack->name_byte_count - t->name_byte_offset) {
            return false;
        }
        if (i != 0 && name_order(pack->name_bytes + t[-1].name_byte_offset, t[-1].name_byte_count, pack->name_bytes + t->name_byte_offset,
                                 t->name_byte_count) >= 0) {
            return false;
        }
    }
    return true;
}

static const struct pack_tensor *tensor_named(const struct exl3_pack_view *pack, const char *name, uint32_t name_count)
{
    uint32_t low = 0, high = pack->tensor_count;
    while (low < high) {
        const uint32_t middle = low + (high - low) / 2u;
        const struct pack_tensor *t = &pack->tensors[middle];
        const int order = name_order(pack->name_bytes + t->name_byte_offset, t->name_byte_count, name, name_count);
        if (order == 0) {
            return t;
        }
        if (order < 0) {
            low = middle + 1u;
        } else {
            high = middle;
        }
    }
    return NULL;
}

/* the routed matrices of one layer and kind by width: each is an EXL3 matrix of the kind's shape */
static bool pack_counts(struct check *check, const struct exl3_pack_view *pack, const struct exl3_descriptor_matrix *matrix, uint32_t layer,
                        uint32_t experts, uint64_t counts[WIDTH_KINDS])
{
    for (uint32_t expert = 0; expert < experts; expert++) {
        char name[160];
        const int length = snprintf(name, sizeof name, "layers.%" PRIu32 ".ffn.experts.%" PRIu32 ".%s.weight", layer, expert, matrix->kind);
        const struct pack_tensor *t = length > 0 && (size_t)length < sizeof name ? tensor_named(pack, name, (uint32_t)length) : NULL;
        const uint32_t bits_x2 = t != NULL ? exl3_bits_x2(t->bits_per_weight) : 0u;
        if (t == NULL || t->weight_format != WEIGHT_FORMAT_EXL3 || t->dimension_count != 2u || t->dimensions[0] != matrix->outputs ||
            t->dimensions[1] != matrix->inputs || bits_x2 < NARROWEST || bits_x2 >= WIDTH_KINDS) {
            return fail(check, STATUS_INVALID_ARGUMENT, "the pack has no EXL3 matrix %s of %" PRIu32 " outputs by %" PRIu32 " inputs", name,
                        matrix->outputs, matrix->inputs);
        }
        counts[bits_x2]++;
    }
    return true;
}

/* ---- the rules by member ---- */

static void kinds_of(const struct exl3_descriptor_model *model, const char *kinds_out[EXL3_DESCRIPTOR_MATRIX_KINDS])
{
    for (uint32_t k = 0; k < EXL3_DESCRIPTOR_MATRIX_KINDS; k++) {
        kinds_out[k] = model->matrices[k].kind;
    }
}

static bool experts_rule(struct check *check, uint32_t experts, const struct exl3_descriptor_model *model)
{
    static const char *const names[] = {"layers", "experts_per_layer", "hidden", "intermediate", "matrices"};
    const uint64_t wanted[] = {model->layers, model->experts_per_layer, model->hidden, model->intermediate};
    uint32_t found[5], shapes[EXL3_DESCRIPTOR_MATRIX_KINDS];
    const char *kinds[EXL3_DESCRIPTOR_MATRIX_KINDS];
    kinds_of(model, kinds);
    if (!members_exactly(check, experts, "experts", names, 5, found)) {
        return false;
    }
    for (uint32_t i = 0; i < 4u; i++) {
        char field[64];
        (void)snprintf(field, sizeof field, "experts.%s", names[i]);
        if (!whole_number_is(check, found[i], field, wanted[i], "the model's")) {
            return false;
        }
    }
    if (!members_exactly(check, found[4], "experts.matrices", kinds, EXL3_DESCRIPTOR_MATRIX_KINDS, shapes)) {
        return false;
    }
    for (uint32_t k = 0; k < EXL3_DESCRIPTOR_MATRIX_KINDS; k++) {
        char field[160];
        (void)snprintf(field, sizeof field, "experts.matrices.%s", kinds[k]);
        const uint64_t sizes[2] = {model->matrices[k].outputs, model->matrices[k].inputs};
        if (!is_kind(check, shapes[k], JSON_TREE_ARRAY) || check->tree->nodes[shapes[k]].child_count != 2u) {
            /* a first size that differs is named as such, as the reference names it, before the count of sizes */
            const uint32_t first = is_kind(check, shapes[k], JSON_TREE_ARRAY) ? check->tree->nodes[shapes[k]].child : JSON_TREE_NONE;
            uint32_t at = 0;
            for (uint32_t item = first; item != JSON_TREE_NONE && at < 2u; item = check->tree->nodes[item].next, at++) {
                if (!whole_number_is(check, item, field, sizes[at], "the model's")) {
                    return false;
                }
            }
            return fail(check, STATUS_INVALID_ARGUMENT, "%s: not [outputs, inputs]", field);
        }
        uint32_t item = check->tree->nodes[shapes[k]].child;
        for (uint32_t at = 0; at < 2u; at++, item = check->tree->nodes[item].next) {
            if (!whole_number_is(check, item, field, sizes[at], "the model's")) {
                return false;
            }
        }
    }
    return true;
}

/* widths against the pack: each layer once, each kind's counts the pack's; on the way the summary's two tables are
 * counted: the matrices by width, the layers by their one width (MIXED for more than one) */
static bool widths_rule(struct check *check, uint32_t widths, const struct exl3_pack_view *pack, const struct exl3_descriptor_model *model,
                        uint64_t matrices[WIDTH_KINDS], uint64_t layers[WIDTH_KINDS])
{
    const char *kinds[EXL3_DESCRIPTOR_MATRIX_KINDS];
    kinds_of(model, kinds);
    if (!is_kind(check, widths, JSON_TREE_OBJECT)) {
        return fail(check, STATUS_INVALID_ARGUMENT, "widths: no object");
    }
    const struct json_tree *tree = check->tree;
    uint32_t layer_count = 0;
    for (uint32_t member = tree->nodes[widths].child; member != JSON_TREE_NONE; member = tree->nodes[member].next, layer_count++) {
        uint64_t layer = 0;
        if (!decimal(tree->strings + tree->nodes[member].key_at, tree->nodes[member].key_count, &layer) || layer >= model->layers) {
            const struct shown s = shown_key(check, member);
            return fail(check, STATUS_INVALID_ARGUMENT, "widths: a layer %.*s, but the model's layers are 0 to %" PRIu32, s.count, s.bytes,
                        model->layers - 1u);
        }
        char field[64];
        (void)snprintf(field, sizeof field, "widths.%" PRIu64, layer);
        uint32_t by_kind[EXL3_DESCRIPTOR_MATRIX_KINDS];
        uint64_t in_layer[WIDTH_KINDS] = {0};
        if (!members_exactly(check, member, field, kinds, EXL3_DESCRIPTOR_MATRIX_KINDS, by_kind)) {
            return false;
        }
        for (uint32_t k = 0; k < EXL3_DESCRIPTOR_MATRIX_KINDS; k++) {
            char kind_field[240];
            uint64_t given[WIDTH_KINDS] = {0}, held[WIDTH_KINDS] = {0};
            (void)snprintf(kind_field, sizeof kind_field, "%s.%s", field, kinds[k]);
            if (!width_counts(check, by_kind[k], kind_field, given) ||
                !pack_counts(check, pack, &model->matrices[k], (uint32_t)layer, model->experts_per_layer, held) ||
                !counts_agree(check, kind_field, given, held, "the pack holds")) {
                return false;
            }
            for (uint32_t place = 0; place < WIDTH_KINDS; place++) {
                in_layer[place] += held[place];
            }
        }
        uint32_t distinct = 0, the_one = MIXED;
        for (uint32_t place = NARROWEST; place < WIDTH_KINDS; place++) {
            matrices[place] += in_layer[place];
            if (in_layer[place] != 0) {
                distinct++;
                the_one = place;
            }
        }
        layers[distinct == 1u ? the_one : MIXED]++;
    }
    /* every key is a layer of the model and no key comes twice: as many keys as layers is every layer once */
    return layer_count == model->layers ||
           fail(check, STATUS_INVALID_ARGUMENT, "widths: %" PRIu32 " layers, but the model has %" PRIu32, layer_count, model->layers);
}

/* a file opened for one pass over its bytes */
struct opened_file {
    int descriptor;
    uint64_t size;
};

/* opens what must be a regular file of at most most_bytes; `what` names it in a line */
static bool regular_open(struct check *check, const char *path, const char *what, uint64_t most_bytes, struct opened_file *file_out)
{
    struct stat about;
    /* not blocking: a FIFO at the path must not hold the open before it is seen to be no regular file */
    file_out->descriptor = open(path, O_RDONLY | O_NONBLOCK | O_NOCTTY | O_CLOEXEC);
    if (file_out->descriptor < 0) {
        return fail(check, STATUS_INPUT_OUTPUT_ERROR, "%s: cannot be opened (%s)", what, strerror(errno));
    }
    if (fstat(file_out->descriptor, &about) != 0) {
        const int error = errno;
        (void)close(file_out->descriptor);
        return fail(check, STATUS_INPUT_OUTPUT_ERROR, "%s: cannot be opened (%s)", what, strerror(error));
    }
    if (!S_ISREG(about.st_mode) || (uint64_t)about.st_size > most_bytes) {
        (void)close(file_out->descriptor);
        return fail(check, STATUS_INVALID_ARGUMENT, "%s: no regular file of at most %" PRIu64 " bytes", what, most_bytes);
    }
    file_out->size = (uint64_t)about.st_size;
    return true;
}

/* one pass over an opened file, which is closed: its SHA-256, and its bytes into `kept` (size + 1 bytes, a NUL behind
 * them) when that is not NULL; else a piece at a time through a buffer of the pass's own */
static bool hashed_through(struct check *check, struct opened_file *file, const char *what, char *kept, unsigned char digest_out[SHA256_DIGEST_BYTES])
{
    char *piece = kept != NULL ? NULL : malloc(HASH_PIECE_BYTES);
    struct sha256_stream stream;
    uint64_t taken = 0;
    bool is_whole = kept != NULL || piece != NULL;
    const bool has_memory = is_whole;
    sha256_begin(&stream);
    while (is_whole && taken < file->size) {
        char *into = kept != NULL ? kept + taken : piece;
        const uint64_t left = file->size - taken;
        const ssize_t got = read(file->descriptor, into, left < HASH_PIECE_BYTES ? (size_t)left : HASH_PIECE_BYTES);
        is_whole = got > 0;
        if (is_whole) {
            sha256_feed(&stream, into, (uint64_t)got);
            taken += (uint64_t)got;
        }
    }
    (void)close(file->descriptor);
    free(piece);
    if (!has_memory) {
        return fail(check, STATUS_OUT_OF_MEMORY, "%s: no memory to read it through", what);
    }
    if (!is_whole) {
        return fail(check, STATUS_INPUT_OUTPUT_ERROR, "%s: cannot be read whole", what);
    }
    if (kept != NULL) {
        kept[file->size] = '\0';
    }
    sha256_finish(&stream, digest_out);
    return true;
}

/* quality: none (only with the opt-in), established by a reference, or recorded by a capture whose digest holds; its
 * words for the line of a descriptor that holds */
static bool quality_rule(struct check *check, uint32_t quality, const char *map, bool admits_unrated, char *words_out, size_t words_bytes)
{
    static const char *const statuses[3] = {"none", "established", "recorded"};
    static const char *const members[3][3] = {{"status"}, {"status", "reference"}, {"status", "record", "sha256"}};
    if (!is_kind(check, quality, JSON_TREE_OBJECT)) {
        const struct shown s = shown_value(check, quality);
        return fail(check, STATUS_INVALID_ARGUMENT, "quality: %.*s is no object", s.count, s.bytes);
    }
    const uint32_t status_node = json_tree_member(check->tree, quality, "status");
    if (status_node == JSON_TREE_NONE) {
        return fail(check, STATUS_INVALID_ARGUMENT, "quality: the member status is missing");
    }
    uint32_t status = 0;
    while (status < 3u && !json_tree_string_is(check->tree, status_node, statuses[status])) {
        status++;
    }
    if (status == 3u) {
        const struct shown s = shown_value(check, status_node);
        return fail(check, STATUS_UNSUPPORTED, "quality.status: %.*s; this build serves \"none\", \"established\" and \"recorded\"", s.count, s.bytes);
    }
    uint32_t found[3];
    if (!members_exactly(check, quality, "quality", members[status], status + 1u, found)) {
        return false;
    }
    if (status == 0u) {
        if (!admits_unrated) {
            return fail(check, STATUS_UNSUPPORTED,
                        "quality: \"none\": nothing measured or qualified covers the map %s; it is served only with " EXL3_DESCRIPTOR_OPT_IN
                        " (no quality claim)",
                        map);
        }
        (void)snprintf(words_out, words_bytes, "none (" EXL3_DESCRIPTOR_OPT_IN ": no quality claim)");
        return true;
    }
    const char *text = NULL;
    uint32_t text_count = 0;
    if (!is_text(check, found[1], status == 1u ? "quality.reference" : "quality.record", &text, &text_count)) {
        return false;
    }
    if (status == 1u) {
        (void)snprintf(words_out, words_bytes, "established (%.*s)", (int)(text_count < 900u ? text_count : 900u), text);
        return true;
    }
    char record[PATH_MAX], named[PATH_MAX + 32];
    if (text[0] != '/' || text_count >= sizeof record) {
        const struct shown s = shown_value(check, found[1]);
        return fail(check, STATUS_INVALID_ARGUMENT, "quality.record: %.*s is no absolute path", s.count, s.bytes);
    }
    memcpy(record, text, text_count);
    record[text_count] = '\0';
    (void)snprintf(named, sizeof named, "quality.record %s", record);
    struct opened_file capture;
    unsigned char capture_digest[SHA256_DIGEST_BYTES];
    if (!regular_open(check, record, named, (uint64_t)INT64_MAX, &capture) || !hashed_through(check, &capture, named, NULL, capture_digest) ||
        !digest_is(check, found[2], "quality.sha256", capture_digest, "the record's")) {
        return false;
    }
    (void)snprintf(words_out, words_bytes, "recorded (%s)", record);
    return true;
}

/* every rule, in the order of the file's members; the line of a descriptor that holds once all do */
static bool descriptor_rules(struct check *check, const unsigned char file_digest[SHA256_DIGEST_BYTES], const char *map, const struct exl3_pack_view *pack,
                             const struct exl3_descriptor_model *model, const char *tables, uint64_t table_byte_count, bool admits_unrated)
{
    const struct json_tree *tree = check->tree;
    if (tree->nodes[0].kind != JSON_TREE_OBJECT) {
        return fail(check, STATUS_INVALID_ARGUMENT, "the file is not one JSON object");
    }
    if (tree->repeats_a_key) {
        return fail(check, STATUS_INVALID_ARGUMENT, "an object of the file has a key twice");
    }
    /* the version first: a later format is named as such, not by the members it adds */
    const uint32_t version = json_tree_member(tree, 0, "format_version");
    uint64_t number = 0;
    if (version == JSON_TREE_NONE) {
        return fail(check, STATUS_INVALID_ARGUMENT, "the member format_version is missing");
    }
    if (tree->nodes[version].kind != JSON_TREE_NUMBER ||
        !decimal(tree->text + tree->nodes[version].begin, tree->nodes[version].end - tree->nodes[version].begin, &number) ||
        number != DESCRIPTOR_FORMAT_VERSION) {
        const struct shown s = shown_value(check, version);
        return fail(check, STATUS_UNSUPPORTED, "format_version: %.*s; this build reads version %u", s.count, s.bytes, DESCRIPTOR_FORMAT_VERSION);
    }
    enum { ROOT_VERSION, ROOT_MAP, ROOT_ARCHITECTURE, ROOT_QUANTISER, ROOT_CODEBOOK, ROOT_TABLES, ROOT_EXPERTS, ROOT_WIDTHS, ROOT_SUMMARY, ROOT_QUALITY, ROOT_COUNT };
    static const char *const root_names[ROOT_COUNT] = {"format_version", "map",    "architecture",   "quantiser", "codebook", "front_end_tables_sha256",
                                                       "experts",        "widths", "widths_summary", "quality"};
    static const char *const map_names[] = {"logical_bytes", "pack_header_digest", "file", "sha256", "manifest_bytes", "native_pack_header_digest"};
    static const char *const architecture_names[] = {"model_type", "architectures", "config_sha256"};
    static const char *const quantiser_names[] = {"source", "index_sha256", "quantization_config_sha256"};
    static const char *const codebook_names[] = {"mul1_multiplier"};
    static const char *const summary_names[] = {"matrices", "layers"};
    uint32_t root[ROOT_COUNT], in_map[6], in_architecture[3], in_quantiser[3], in_codebook[1], in_summary[2];
    if (!members_exactly(check, 0, "the descriptor", root_names, ROOT_COUNT, root) ||
        !members_exactly(check, root[ROOT_MAP], "map", map_names, 6, in_map) ||
        !whole_number_is(check, in_map[0], "map.logical_bytes", pack->file_byte_count, "the pack's size") ||
        !whole_number_is(check, in_map[1], "map.pack_header_digest", pack->header_digest, "the pack's") ||
        !members_exactly(check, root[ROOT_ARCHITECTURE], "architecture", architecture_names, 3, in_architecture)) {
        return false;
    }
    if (!json_tree_string_is(tree, in_architecture[0], model->model_type)) {
        const struct shown s = shown_value(check, in_architecture[0]);
        return fail(check, STATUS_UNSUPPORTED, "architecture.model_type: %.*s, but the model is \"%s\"", s.count, s.bytes, model->model_type);
    }
    const char *source = NULL;
    uint32_t source_count = 0;
    if (!members_exactly(check, root[ROOT_QUANTISER], "quantiser", quantiser_names, 3, in_quantiser) ||
        !is_text(check, in_quantiser[0], "quantiser.source", &source, &source_count) ||
        !members_exactly(check, root[ROOT_CODEBOOK], "codebook", codebook_names, 1, in_codebook)) {
        return false;
    }
    char multiplier[16];
    (void)snprintf(multiplier, sizeof multiplier, "0x%08" PRIX32, (uint32_t)EXL3_MUL1_MULTIPLIER);
    if (!json_tree_string_is(tree, in_codebook[0], multiplier)) {
        const struct shown s = shown_value(check, in_codebook[0]);
        return fail(check, STATUS_UNSUPPORTED, "codebook.mul1_multiplier: %.*s, but this build's kernels decode with \"%s\"", s.count, s.bytes, multiplier);
    }
    if (tables != NULL && !is_kind(check, root[ROOT_TABLES], JSON_TREE_NULL)) {
        unsigned char digest[SHA256_DIGEST_BYTES];
        anemone_sha256(tables, table_byte_count, digest);
        if (!digest_is(check, root[ROOT_TABLES], "front_end_tables_sha256", digest, "the tables'")) {
            return false;
        }
    }
    uint64_t matrices[WIDTH_KINDS] = {0}, layers[WIDTH_KINDS] = {0}, given[WIDTH_KINDS] = {0}, given_layers[WIDTH_KINDS] = {0};
    uint64_t exl3_matrices = 0;
    for (uint32_t t = 0; t < pack->tensor_count; t++) {
        exl3_matrices += pack->tensors[t].weight_format == WEIGHT_FORMAT_EXL3 ? 1u : 0u;
    }
    const uint64_t routed = (uint64_t)model->layers * model->experts_per_layer * EXL3_DESCRIPTOR_MATRIX_KINDS;
    char quality_words[PATH_MAX + 64];
    if (!experts_rule(check, root[ROOT_EXPERTS], model) || !widths_rule(check, root[ROOT_WIDTHS], pack, model, matrices, layers)) {
        return false;
    }
    if (exl3_matrices != routed) {
        return fail(check, STATUS_INVALID_ARGUMENT, "the pack has %" PRIu64 " EXL3 matrices, but the model's routed experts are %" PRIu64,
                    exl3_matrices, routed);
    }
    if (!members_exactly(check, root[ROOT_SUMMARY], "widths_summary", summary_names, 2, in_summary) ||
        !width_counts(check, in_summary[0], "widths_summary.matrices", given) ||
        !counts_agree(check, "widths_summary.matrices", given, matrices, "widths gives") ||
        !width_counts(check, in_summary[1], "widths_summary.layers", given_layers) ||
        !counts_agree(check, "widths_summary.layers", given_layers, layers, "widths gives") ||
        !quality_rule(check, root[ROOT_QUALITY], map, admits_unrated, quality_words, sizeof quality_words)) {
        return false;
    }
    char widths_words[WIDTH_KINDS * 32] = "", sidecar_digest[2 * SHA256_DIGEST_BYTES + 1];
    size_t used = 0;
    for (uint32_t place = NARROWEST; place < WIDTH_KINDS; place++) {
        if (matrices[place] != 0) {
            char name[WIDTH_NAME_BYTES];
            width_name(place, name);
            const int written = snprintf(widths_words + used, sizeof widths_words - used, "%s%s %" PRIu64, used != 0 ? ", " : "", name, matrices[place]);
            used += written > 0 ? (size_t)written : 0u;
        }
    }
    hexadecimal(file_digest, sidecar_digest);
    (void)fprintf(stderr, "anemone: exl3 descriptor %s (sha256 %s) holds: model %s, quantiser %.*s, widths %s, quality %s\n", check->sidecar,
                  sidecar_digest, model->model_type, (int)(source_count < 400u ? source_count : 400u), source, widths_words, quality_words);
    return true;
}

/* no sidecar: the open pack is served by default when the model lists it as established (its header digest and its
 * size), else only on the opt-in */
static bool absent_rule(struct check *check, const struct exl3_pack_view *pack, const struct exl3_descriptor_model *model, bool admits_unrated)
{
    const struct exl3_established_pack *listed = NULL;
    for (uint32_t i = 0; listed == NULL && i < model->established_count; i++) {
        if (model->established[i].header_digest == pack->header_digest && model->established[i].file_byte_count == pack->file_byte_count) {
            listed = &model->established[i];
        }
    }
    if (listed == NULL && !admits_unrated) {
        return fail(check, STATUS_UNSUPPORTED,
                    "no such file, and the model does not list the pack (header digest %" PRIu64 ", %" PRIu64
                    " bytes) as established: it is served only with " EXL3_DESCRIPTOR_OPT_IN " (no quality claim)",
                    pack->header_digest, pack->file_byte_count);
    }
    (void)fprintf(stderr, "anemone: exl3 descriptor %s: no such file; %s%s (header digest %" PRIu64 ", %" PRIu64 " bytes) is served %s\n", check->sidecar,
                  listed != NULL ? "the established pack " : "a pack the model does not list as established", listed != NULL ? listed->name : "",
                  pack->header_digest, pack->file_byte_count,
                  listed != NULL ? "by default" : "on " EXL3_DESCRIPTOR_OPT_IN " (no quality claim)");
    return true;
}

/* what the check needs of its arguments before it looks at any file */
static bool arguments_are_usable(const char *map_path, const struct exl3_pack_view *pack, const struct exl3_descriptor_model *model, const char *tables,
                                 uint64_t table_byte_count)
{
    if (map_path == NULL || pack == NULL || model == NULL || (table_byte_count != 0 && tables == NULL)) {
        return false;
    }
    bool usable = model->model_type != NULL && model->layers != 0 && model->experts_per_layer != 0 &&
                  (model->established_count == 0 || model->established != NULL);
    for (uint32_t k = 0; usable && k < EXL3_DESCRIPTOR_MATRIX_KINDS; k++) {
        usable = model->matrices[k].kind != NULL;
    }
    return usable;
}

result_status exl3_descriptor_check(const char *map_path, const struct exl3_pack_view *pack, const struct exl3_descriptor_model *model,
                                    const char *tables, uint64_t table_byte_count, bool admits_unrated)
{
    if (!arguments_are_usable(map_path, pack, model, tables, table_byte_count)) {
        return STATUS_INVALID_ARGUMENT;
    }
    if (!view_is_sound(pack)) {
        REFUSE("exl3 descriptor: the pack's tensor records are not sorted by name inside their name bytes");
        return STATUS_INVALID_ARGUMENT;
    }
    /* the sidecar lies beside the map the path leads to; beside the path as given when it leads nowhere */
    char resolved[PATH_MAX], sidecar[PATH_MAX];
    const char *map = realpath(map_path, resolved);
    if (map == NULL) {
        map = map_path;
    }
    if (strlen(map) + sizeof EXL3_DESCRIPTOR_SUFFIX > sizeof sidecar) {
        REFUSE("exl3 descriptor: the map's path %.200s... leaves no room for its sidecar's", map);
        return STATUS_INVALID_ARGUMENT;
    }
    (void)snprintf(sidecar, sizeof sidecar, "%s%s", map, EXL3_DESCRIPTOR_SUFFIX);
    struct check check = {.sidecar = sidecar, .status = STATUS_OK};
    struct stat entry;
    /* nothing at the path, not even a link (a link to nothing fails at its open), or nothing can be: a name too long */
    const bool is_absent = lstat(sidecar, &entry) != 0 && (errno == ENOENT || errno == ENAMETOOLONG);
    if (is_absent) {
        (void)absent_rule(&check, pack, model, admits_unrated);
        return check.status;
    }
    struct opened_file file;
    unsigned char digest[SHA256_DIGEST_BYTES];
    if (!regular_open(&check, sidecar, "the file", EXL3_DESCRIPTOR_MOST_BYTES, &file)) {
        return check.status;
    }
    char *text = malloc((size_t)file.size + 1u);
    if (text == NULL) {
        (void)close(file.descriptor);
        (void)fail(&check, STATUS_OUT_OF_MEMORY, "the file: no memory to read it into");
        return check.status;
    }
    struct json_tree tree = {0};
    if (hashed_through(&check, &file, "the file", text, digest)) {
        switch (json_tree_read(text, (size_t)file.size, &tree)) {
        case JSON_TREE_NO_MEMORY: (void)fail(&check, STATUS_OUT_OF_MEMORY, "no memory to check it in"); break;
        case JSON_TREE_NOT_JSON: (void)fail(&check, STATUS_INVALID_ARGUMENT, "the file is not one JSON object"); break;
        case JSON_TREE_READ:
            check.tree = &tree;
            if (!descriptor_rules(&check, digest, map, pack, model, tables, table_byte_count, admits_unrated) && check.status == STATUS_OK) {
                check.status = STATUS_INVALID_ARGUMENT; /* not reached: every rule that fails leaves its status */
            }
            json_tree_free(&tree);
            break;
        }
    }
    free(text);
    return check.status;
}

result_status exl3_descriptor_tc_check(const char *model_name, const struct exl3_descriptor_model *model, uint32_t ranks, uint32_t rotation)
{
    (void)rotation;
    if (model_name == NULL || model == NULL || ranks == 0) {
        return STATUS_INVALID_ARGUMENT;
    }
    static const char line[] = "exl3 descriptor: the fused EXL3 kernels and the model %s: ";
    const struct {
        const char *field;
        uint32_t value, most;
    } counted[] = {{"routes_per_row", model->routes_per_row, ROUTER_MOST_PICKS}, {"experts.experts_per_layer", model->experts_per_layer, ROUTER_MOST_EXPERTS}};
    for (size_t i = 0; i < sizeof counted / sizeof counted[0]; i++) {
        if (counted[i].value == 0 || counted[i].value > counted[i].most) {
            char begun[256];
            (void)snprintf(begun, sizeof begun, line, model_name);
            REFUSE("%s%s is %" PRIu32 ", and the job table takes 1 to %" PRIu32, begun, counted[i].field, counted[i].value, counted[i].most);
            return STATUS_UNSUPPORTED;
        }
    }
    for (uint32_t rank = 0; rank < ranks; rank++) {
        struct bb_exl3_output_shard_plan plan;
        char begun[256];
        (void)snprintf(begun, sizeof begun, line, model_name);
        if (bb_exl3_output_shard_prepare(model->hidden, model->intermediate, EXL3_K3, ranks, rank, BB_EXL3_REFERENCE_ORDER, &plan) != STATUS_OK) {
            REFUSE("%sexperts.intermediate %" PRIu32 " has no split over %" PRIu32 " ranks", begun, model->intermediate, ranks);
            return STATUS_UNSUPPORTED;
        }
        const char *why = exl3_tc_geometry_refusal(model->hidden, plan.gate_up.output_count);
        if (why != NULL) {
            REFUSE("%sexperts.hidden %" PRIu32 " with rank %" PRIu32 "'s %" PRIu32 " of experts.intermediate %" PRIu32 ": %s", begun, model->hidden, rank,
                   plan.gate_up.output_count, model->intermediate, why);
            return STATUS_UNSUPPORTED;
        }
    }
    return STATUS_OK;
}
