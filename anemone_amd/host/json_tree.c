/* json_tree.c -- a JSON text into a tree of nodes: a recursive-descent reader of json.loads's grammar (json_tree.h). The
 * reference's descriptor check walks spans of the text through its own reader (source/json.h:5-13, used at
 * source/exl3_descriptor.c:744-755); here the text is read once, every string unescaped once, and the check works on
 * nodes. */
#include <stdlib.h>
#include <string.h>

#include "json_tree.h"

struct reader {
    const char *text;
    uint32_t end, at;
    struct json_tree *tree;
    uint32_t node_capacity, string_used;
    bool no_memory;
};

static void skip_spaces(struct reader *r)
{
    while (r->at < r->end && (r->text[r->at] == ' ' || r->text[r->at] == '\t' || r->text[r->at] == '\n' || r->text[r->at] == '\r')) {
        r->at++;
    }
}

static uint32_t node_new(struct reader *r, uint32_t kind)
{
    struct json_tree *tree = r->tree;
    if (tree->node_count == r->node_capacity) {
        const uint32_t capacity = r->node_capacity != 0 ? 2u * r->node_capacity : 64u;
        struct json_tree_node *grown = realloc(tree->nodes, (size_t)capacity * sizeof *grown);
        if (grown == NULL) {
            r->no_memory = true;
            return JSON_TREE_NONE;
        }
        tree->nodes = grown;
        r->node_capacity = capacity;
    }
    struct json_tree_node *node = &tree->nodes[tree->node_count];
    memset(node, 0, sizeof *node);
    node->kind = kind;
    node->begin = r->at;
    node->child = node->next = JSON_TREE_NONE;
    return tree->node_count++;
}

static bool takes(struct reader *r, const char *word)
{
    const size_t length = strlen(word);
    if (r->end - r->at < length || memcmp(r->text + r->at, word, length) != 0) {
        return false;
    }
    r->at += (uint32_t)length;
    return true;
}

static int hex_digit(char c)
{
    return c >= '0' && c <= '9' ? c - '0' : c >= 'a' && c <= 'f' ? c - 'a' + 10 : c >= 'A' && c <= 'F' ? c - 'A' + 10 : -1;
}

/* four hexadecimal digits at the cursor */
static bool hex_unit(struct reader *r, uint32_t *unit_out)
{
    uint32_t unit = 0;
    if (r->end - r->at < 4u) {
        return false;
    }
    for (unsigned i = 0; i < 4u; i++) {
        const int digit = hex_digit(r->text[r->at + i]);
        if (digit < 0) {
            return false;
        }
        unit = unit << 4 | (uint32_t)digit;
    }
    r->at += 4u;
    *unit_out = unit;
    return true;
}

static void put_code_point(struct reader *r, uint32_t c)
{
    char *out = r->tree->strings + r->string_used;
    if (c < 0x80u) {
        out[0] = (char)c;
        r->string_used += 1u;
    } else if (c < 0x800u) {
        out[0] = (char)(0xC0u | c >> 6);
        out[1] = (char)(0x80u | (c & 0x3Fu));
        r->string_used += 2u;
    } else if (c < 0x10000u) {
        out[0] = (char)(0xE0u | c >> 12);
        out[1] = (char)(0x80u | (c >> 6 & 0x3Fu));
        out[2] = (char)(0x80u | (c & 0x3Fu));
        r->string_used += 3u;
    } else {
        out[0] = (char)(0xF0u | c >> 18);
        out[1] = (char)(0x80u | (c >> 12 & 0x3Fu));
        out[2] = (char)(0x80u | (c >> 6 & 0x3Fu));
        out[3] = (char)(0x80u | (c & 0x3Fu));
        r->string_used += 4u;
    }
}

/* the bytes of one UTF-8 sequence at the cursor, copied as they are: 0 for bytes that are none */
static unsigned utf8_sequence(const struct reader *r)
{
    const unsigned char *s = (const unsigned char *)r->text + r->at;
    const uint32_t left = r->end - r->at;
    const unsigned length = s[0] < 0x80u ? 1u : (s[0] & 0xE0u) == 0xC0u ? 2u : (s[0] & 0xF0u) == 0xE0u ? 3u : (s[0] & 0xF8u) == 0xF0u ? 4u : 0u;
    if (length == 0u || left < length) {
        return 0u;
    }
    uint32_t c = length == 1u ? s[0] : s[0] & (0xFFu >> (length + 1u));
    for (unsigned i = 1; i < length; i++) {
        if ((s[i] & 0xC0u) != 0x80u) {
            return 0u;
        }
        c = c << 6 | (s[i] & 0x3Fu);
    }
    static const uint32_t least[5] = {0, 0, 0x80u, 0x800u, 0x10000u};
    if (c < least[length] || c > 0x10FFFFu || (c >= 0xD800u && c <= 0xDFFFu)) {
        return 0u;
    }
    return length;
}

/* a string at the cursor (on its opening quote), unescaped behind what the strings hold */
static bool read_string(struct reader *r, uint32_t *at_out, uint32_t *count_out)
{
    const uint32_t start = r->string_used;
    r->at++;
    while (r->at < r->end) {
        const unsigned char c = (unsigned char)r->text[r->at];
        if (c == '"') {
            r->at++;
            *at_out = start;
            *count_out = r->string_used - start;
            return true;
        }
        if (c < 0x20u) {
            return false;
        }
        if (c != '\\') {
            const unsigned length = utf8_sequence(r);
            if (length == 0u) {
                return false;
            }
            memcpy(r->tree->strings + r->string_used, r->text + r->at, length);
            r->string_used += length;
            r->at += length;
            continue;
        }
        if (r->end - r->at < 2u) {
            return false;
        }
        const char escape = r->text[r->at + 1u];
        r->at += 2u;
        static const char short_escapes[] = "\"\\/bfnrt", short_values[] = "\"\\/\b\f\n\r\t";
        const char *found = escape != '\0' ? strchr(short_escapes, escape) : NULL;
        if (found != NULL) {
            r->tree->strings[r->string_used++] = short_values[found - short_escapes];
            continue;
        }
        uint32_t unit = 0, low = 0;
        if (escape != 'u' || !hex_unit(r, &unit)) {
            return false;
        }
        if (unit >= 0xD800u && unit <= 0xDBFFu) { /* the high half: the low half follows, escaped too */
            if (!takes(r, "\\u") || !hex_unit(r, &low) || low < 0xDC00u || low > 0xDFFFu) {
                return false;
            }
            unit = 0x10000u + ((unit - 0xD800u) << 10) + (low - 0xDC00u);
        } else if (unit >= 0xDC00u && unit <= 0xDFFFu) {
            return false;
        }
        put_code_point(r, unit);
    }
    return false;
}

static bool digits(struct reader *r, uint32_t *count_out)
{
    const uint32_t start = r->at;
    while (r->at < r->end && r->text[r->at] >= '0' && r->text[r->at] <= '9') {
        r->at++;
    }
    *count_out = r->at - start;
    return r->at > start;
}

static bool read_number(struct reader *r)
{
    uint32_t count = 0;
    if (r->at < r->end && r->text[r->at] == '-') {
        r->at++;
        if (takes(r, "Infinity")) {
            return true;
        }
    }
    if (r->at < r->end && r->text[r->at] == '0') {
        r->at++;
        count = 1u;
    } else if (!digits(r, &count)) {
        return false;
    }
    bool is_integer = true;
    uint32_t more = 0;
    if (r->at < r->end && r->text[r->at] == '.') {
        r->at++;
        is_integer = false;
        if (!digits(r, &more)) {
            return false;
        }
    }
    if (r->at < r->end && (r->text[r->at] == 'e' || r->text[r->at] == 'E')) {
        r->at++;
        is_integer = false;
        if (r->at < r->end && (r->text[r->at] == '+' || r->text[r->at] == '-')) {
            r->at++;
        }
        if (!digits(r, &more)) {
            return false;
        }
    }
    return !is_integer || count <= JSON_TREE_MOST_INTEGER_DIGITS;
}

struct key_order {
    const struct json_tree *tree;
};

static int by_key(const void *left, const void *right, void *context)
{
    const struct json_tree *tree = ((const struct key_order *)context)->tree;
    const struct json_tree_node *a = &tree->nodes[*(const uint32_t *)left], *b = &tree->nodes[*(const uint32_t *)right];
    const uint32_t shared = a->key_count < b->key_count ? a->key_count : b->key_count;
    const int order = shared != 0 ? memcmp(tree->strings + a->key_at, tree->strings + b->key_at, shared) : 0;
    return order != 0 ? order : a->key_count < b->key_count ? -1 : a->key_count > b->key_count ? 1 : 0;
}

/* whether two members of the object have the same key: its members sorted by key, then neighbours compared */
static bool object_repeats(struct reader *r, uint32_t object)
{
    const struct json_tree *tree = r->tree;
    const uint32_t count = tree->nodes[object].child_count;
    if (count < 2u) {
        return false;
    }
    uint32_t *members = malloc((size_t)count * sizeof *members);
    if (members == NULL) {
        r->no_memory = true;
        return false;
    }
    uint32_t filled = 0;
    for (uint32_t member = tree->nodes[object].child; member != JSON_TREE_NONE; member = tree->nodes[member].next) {
        members[filled++] = member;
    }
    struct key_order order = {tree};
    qsort_r(members, count, sizeof *members, by_key, &order);
    bool repeats = false;
    for (uint32_t i = 1; i < count && !repeats; i++) {
        repeats = by_key(&members[i - 1u], &members[i], &order) == 0;
    }
    free(members);
    return repeats;
}

static uint32_t read_value(struct reader *r, uint32_t depth);

/* the items of an array or the members of an object, the cursor behind its opening bracket */
static bool read_children(struct reader *r, uint32_t parent, bool keyed, char closing, uint32_t depth)
{
    uint32_t last = JSON_TREE_NONE;
    skip_spaces(r);
    if (r->at < r->end && r->text[r->at] == closing) {
        r->at++;
        return true;
    }
    for (;;) {
        uint32_t key_begin = 0, key_end = 0, key_at = 0, key_count = 0;
        skip_spaces(r);
        if (keyed) {
            key_begin = r->at;
            if (r->at >= r->end || r->text[r->at] != '"' || !read_string(r, &key_at, &key_count)) {
                return false;
            }
            key_end = r->at;
            skip_spaces(r);
            if (r->at >= r->end || r->text[r->at] != ':') {
                return false;
            }
            r->at++;
        }
        const uint32_t child = read_value(r, depth + 1u);
        if (child == JSON_TREE_NONE) {
            return false;
        }
        struct json_tree_node *nodes = r->tree->nodes;
        nodes[child].key_begin = key_begin;
        nodes[child].key_end = key_end;
        nodes[child].key_at = key_at;
        nodes[child].key_count = key_count;
        if (last == JSON_TREE_NONE) {
            nodes[parent].child = child;
        } else {
            nodes[last].next = child;
        }
        nodes[parent].child_count++;
        last = child;
        skip_spaces(r);
        if (r->at < r->end && r->text[r->at] == ',') {
            r->at++;
            continue;
        }
        if (r->at < r->end && r->text[r->at] == closing) {
            r->at++;
            return true;
        }
        return false;
    }
}

/* one value at the cursor, spaces before it skipped: its node, or JSON_TREE_NONE */
static uint32_t read_value(struct reader *r, uint32_t depth)
{
    skip_spaces(r);
    if (r->at >= r->end || r->no_memory) {
        return JSON_TREE_NONE;
    }
    const char first = r->text[r->at];
    const uint32_t kind = first == '{'   ? JSON_TREE_OBJECT
                          : first == '[' ? JSON_TREE_ARRAY
                          : first == '"' ? JSON_TREE_STRING
                          : first == 't' ? JSON_TREE_TRUE
                          : first == 'f' ? JSON_TREE_FALSE
                          : first == 'n' ? JSON_TREE_NULL
                                         : JSON_TREE_NUMBER;
    const uint32_t node = node_new(r, kind);
    if (node == JSON_TREE_NONE) {
        return JSON_TREE_NONE;
    }
    bool is_read;
    if (kind == JSON_TREE_OBJECT || kind == JSON_TREE_ARRAY) {
        r->at++;
        is_read = depth < JSON_TREE_MOST_DEPTH && read_children(r, node, kind == JSON_TREE_OBJECT, kind == JSON_TREE_OBJECT ? '}' : ']', depth);
        if (is_read && kind == JSON_TREE_OBJECT && object_repeats(r, node)) {
            r->tree->repeats_a_key = true;
        }
    } else if (kind == JSON_TREE_STRING) {
        uint32_t at = 0, count = 0;
        is_read = read_string(r, &at, &count);
        r->tree->nodes[node].text_at = at;
        r->tree->nodes[node].text_count = count;
    } else if (kind == JSON_TREE_NUMBER) {
        is_read = takes(r, "NaN") || takes(r, "Infinity") || read_number(r);
    } else {
        is_read = takes(r, kind == JSON_TREE_TRUE ? "true" : kind == JSON_TREE_FALSE ? "false" : "null");
    }
    if (!is_read || r->no_memory) {
        return JSON_TREE_NONE;
    }
    r->tree->nodes[node].end = r->at;
    return node;
}

enum json_tree_status json_tree_read(const char *text, size_t byte_count, struct json_tree *tree_out)
{
    struct json_tree tree = {.text = text};
    if (text == NULL || tree_out == NULL || byte_count > UINT32_MAX / 2u) {
        return JSON_TREE_NOT_JSON;
    }
    tree.strings = malloc(byte_count + 4u); /* an unescaped string is never longer than it is written */
    if (tree.strings == NULL) {
        return JSON_TREE_NO_MEMORY;
    }
    struct reader r = {.text = text, .end = (uint32_t)byte_count, .tree = &tree};
    const uint32_t root = read_value(&r, 0);
    skip_spaces(&r);
    if (root == JSON_TREE_NONE || r.at != r.end) {
        json_tree_free(&tree);
        return r.no_memory ? JSON_TREE_NO_MEMORY : JSON_TREE_NOT_JSON;
    }
    *tree_out = tree;
    return JSON_TREE_READ;
}

void json_tree_free(struct json_tree *tree)
{
    if (tree != NULL) {
        free(tree->nodes);
        free(tree->strings);
        tree->nodes = NULL;
        tree->strings = NULL;
        tree->node_count = 0;
    }
}

bool json_tree_key_is(const struct json_tree *tree, uint32_t node, const char *text)
{
    const struct json_tree_node *n = &tree->nodes[node];
    return n->key_end != 0 && n->key_count == strlen(text) && memcmp(tree->strings + n->key_at, text, n->key_count) == 0;
}

bool json_tree_string_is(const struct json_tree *tree, uint32_t node, const char *text)
{
    const struct json_tree_node *n = node != JSON_TREE_NONE ? &tree->nodes[node] : NULL;
    return n != NULL && n->kind == JSON_TREE_STRING && n->text_count == strlen(text) && memcmp(tree->strings + n->text_at, text, n->text_count) == 0;
}

uint32_t json_tree_member(const struct json_tree *tree, uint32_t object, const char *key)
{
    if (object == JSON_TREE_NONE || tree->nodes[object].kind != JSON_TREE_OBJECT) {
        return JSON_TREE_NONE;
    }
    for (uint32_t member = tree->nodes[object].child; member != JSON_TREE_NONE; member = tree->nodes[member].next) {
        if (json_tree_key_is(tree, member, key)) {
            return member;
        }
    }
    return JSON_TREE_NONE;
}
