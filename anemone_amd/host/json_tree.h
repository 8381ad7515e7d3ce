/* json_tree.h -- a JSON text read once into a tree (json_tree.c); private to the library's host sources.
 *
 * The grammar is the one Python's json.loads reads (the reference's source/json.h:5-13 states the same contract for its
 * reader, which the descriptor's check is written over): spaces (space, tab, line feed, carriage return), one value,
 * spaces; objects, arrays, strings with their escapes, numbers (-?int frac? exp?, an integer of at most 4300 digits),
 * true, false, null, NaN, Infinity, -Infinity. Refused besides: bytes in a string that are no UTF-8 (overlong forms,
 * surrogates and code points above U+10FFFF among them), control bytes in a string, an escaped half of a surrogate pair
 * without the other, nesting deeper than JSON_TREE_MOST_DEPTH.
 *
 * A node is a value; an object's members are its children, each with its key. Strings and keys are held unescaped (their
 * bytes may hold NULs: a count goes with them). json_tree_read also says whether any object holds a key twice (json.loads
 * would keep the last: the caller decides). */
#ifndef ANEMONE_HOST_JSON_TREE_H
#define ANEMONE_HOST_JSON_TREE_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#define JSON_TREE_MOST_DEPTH 128u
#define JSON_TREE_MOST_INTEGER_DIGITS 4300u
#define JSON_TREE_NONE UINT32_MAX

enum json_tree_kind { JSON_TREE_NULL, JSON_TREE_TRUE, JSON_TREE_FALSE, JSON_TREE_NUMBER, JSON_TREE_STRING, JSON_TREE_ARRAY, JSON_TREE_OBJECT };

struct json_tree_node {
    uint32_t kind;               /* enum json_tree_kind */
    uint32_t begin, end;         /* the value as it is written: text[begin .. end) */
    uint32_t child, next;        /* the first item or member, the next one of the same parent; JSON_TREE_NONE for none */
    uint32_t child_count;
    uint32_t text_at, text_count; /* a string unescaped: strings[text_at .. + text_count) */
    uint32_t key_begin, key_end; /* a member's key as it is written, quotes included; 0, 0 for an item or the root */
    uint32_t key_at, key_count;  /* and unescaped */
};

struct json_tree {
    const char *text;
    struct json_tree_node *nodes; /* nodes[0] is the document's value */
    char *strings;
    uint32_t node_count;
    bool repeats_a_key;
};

enum json_tree_status { JSON_TREE_READ, JSON_TREE_NOT_JSON, JSON_TREE_NO_MEMORY };

/* text need not end in a NUL and must stay while the tree is used; at most UINT32_MAX / 2 bytes */
enum json_tree_status json_tree_read(const char *text, size_t byte_count, struct json_tree *tree_out);
void json_tree_free(struct json_tree *tree);

/* the member of an object by its key (unescaped bytes), or JSON_TREE_NONE; the first when the object repeats it */
uint32_t json_tree_member(const struct json_tree *tree, uint32_t object, const char *key);
bool json_tree_string_is(const struct json_tree *tree, uint32_t node, const char *text);
bool json_tree_key_is(const struct json_tree *tree, uint32_t node, const char *text);

#endif
