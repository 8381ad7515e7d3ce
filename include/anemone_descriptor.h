/*
 * anemone_descriptor.h -- the check of an EXL3 map's descriptor (the sidecar <map>.descriptor.json the converter writes
 * beside a map) against the open pack's tensor records and the model's geometry, before anything is loaded. Host only:
 * no card, no launch.
 *
 * Replaces source/exl3_descriptor.h:7-93 of the reference (exl3_descriptor_check, exl3_descriptor_tc_check, the model
 * record) with the same names, argument meaning and statuses. The reference reads the pack through its storage engine
 * (include/anemone/pack.h:150-195: pack_open_entry and the accessors); that engine is outside this library, so the
 * check takes what it needs of an open pack as a view: the two header fields the descriptor binds to and the tensor
 * records with their name bytes, in the layout the file stores them (pack.h:68-146). A binding over the reference's
 * pack fills the view from pack_header_of, pack_tensors_of and pack_name_bytes_of without a copy.
 *
 * Rules (exl3_descriptor.h:7-40): the sidecar is the map's real path (the path as given when it does not resolve) with
 * EXL3_DESCRIPTOR_SUFFIX behind it. Nothing there (nor can be: a name over NAME_MAX): the pack is served when the model
 * lists its header digest and size as established, or on admits_unrated; else STATUS_UNSUPPORTED. Otherwise every rule
 * holds or one line on stderr names the sidecar and the field, with STATUS_UNSUPPORTED for a format version, model,
 * codebook or quality this build does not serve, STATUS_INPUT_OUTPUT_ERROR for a file that cannot be read,
 * STATUS_OUT_OF_MEMORY, and STATUS_INVALID_ARGUMENT for every other rule:
 *   a regular file of at most EXL3_DESCRIPTOR_MOST_BYTES holding one JSON object (json.loads's grammar), no key twice
 *   in any object; format_version 1; then exactly the members the converter writes:
 *     map {logical_bytes, pack_header_digest, file, sha256, manifest_bytes, native_pack_header_digest}: the first two the
 *       view's file_byte_count and header_digest;
 *     architecture {model_type, architectures, config_sha256}: model_type the model's;
 *     quantiser {source, index_sha256, quantization_config_sha256}: source a text (a byte other than a space, no NUL);
 *     codebook {mul1_multiplier}: "0x83DCD12D" (EXL3_MUL1_MULTIPLIER as "0x%08X");
 *     front_end_tables_sha256: the tables' SHA-256 when tables were given and the member is not null;
 *     experts {layers, experts_per_layer, hidden, intermediate, matrices {kind: [outputs, inputs]}}: the model's;
 *     widths {layer: {kind: {width: count}}}: every layer 0 .. layers - 1 once (decimal, no leading zero), every kind,
 *       counts at least 1 of "K<n>" / "K<n>.5", equal to what the view's records give: every routed matrix
 *       layers.<layer>.ffn.experts.<expert>.<kind>.weight is an EXL3 matrix of its kind's shape, and the view holds no
 *       other EXL3 matrix;
 *     widths_summary {matrices, layers}: those counts summed by width, and the layers by their one width ("mixed" for a
 *       layer of more than one);
 *     quality: {"status": "none"} only with admits_unrated; {"status": "established", "reference": text};
 *       {"status": "recorded", "record": absolute path, "sha256": that file's, which is read and checked}.
 * On success one line on stderr gives the sidecar, its SHA-256, the quantiser's source, the widths and the quality.
 */
#ifndef ANEMONE_DESCRIPTOR_H
#define ANEMONE_DESCRIPTOR_H

#include <stdbool.h>
#include <stdint.h>

#include "anemone_backend.h"

#ifdef __cplusplus
extern "C" {
#endif

#define EXL3_DESCRIPTOR_SUFFIX ".descriptor.json"
#define EXL3_DESCRIPTOR_MOST_BYTES 1048576u
#define EXL3_DESCRIPTOR_MATRIX_KINDS 3u /* a routed expert's matrices: gate, up, down */
#define EXL3_DESCRIPTOR_OPT_IN "--exl3_unrated_map=1"

/* A tensor record as a pack stores it (include/anemone/pack.h:131-146 of the reference; 64 bytes, little-endian). A
 * translation unit that also includes the reference's pack.h includes it first: its struct is then the one used. */
#ifndef PACK_H
#define PACK_MAXIMUM_DIMENSIONS 4
struct pack_tensor {
    uint64_t byte_offset_in_extent;
    uint64_t byte_count;
    uint32_t extent_index;
    uint32_t name_byte_offset; /* into the name bytes; names are not NUL-terminated */
    uint32_t name_byte_count;
    uint32_t element_type;
    uint32_t dimension_count;
    uint32_t dimensions[PACK_MAXIMUM_DIMENSIONS];
    uint32_t weight_format;   /* enum weight_format_code */
    uint32_t bits_per_weight; /* EXL3: the stored width (K, or 16 K + 8 for a half K) */
    uint32_t reserved_zero[1];
};
#endif
#ifndef __cplusplus
_Static_assert(sizeof(struct pack_tensor) == 64, "a tensor record as the file stores it");
#endif

/* What the check reads of an open pack (pack.h:68-82 header fields; :176-186 accessors). The records are sorted by name
 * as unsigned bytes, a shorter name before a longer one it begins (pack.h:17-18); the check verifies that and that
 * every name lies inside the name bytes before it searches them. */
struct exl3_pack_view {
    uint64_t header_digest, file_byte_count;
    const struct pack_tensor *tensors;
    const char *name_bytes;
    uint32_t tensor_count, name_byte_count;
};

/* exl3_descriptor.h:52-75 */
struct exl3_descriptor_matrix {
    const char *kind; /* layers.<layer>.ffn.experts.<expert>.<kind>.weight */
    uint32_t outputs, inputs;
};
struct exl3_established_pack {
    const char *name;
    uint64_t header_digest, file_byte_count;
};
struct exl3_descriptor_model {
    const char *model_type;
    uint32_t layers, experts_per_layer, hidden, intermediate;
    struct exl3_descriptor_matrix matrices[EXL3_DESCRIPTOR_MATRIX_KINDS];
    const struct exl3_established_pack *established;
    uint32_t established_count;
    uint32_t routes_per_row, cone_first_layer;
};

/* exl3_descriptor.h:77-81. map_path: the map as the run names it; tables: the front end's tables when read, else NULL */
MUST_CHECK result_status exl3_descriptor_check(const char *map_path, const struct exl3_pack_view *pack,
                                               const struct exl3_descriptor_model *model, const char *tables,
                                               uint64_t table_byte_count, bool admits_unrated);

/* exl3_descriptor.h:83-91: the model against the geometry the tensor-core MoE kernels of THIS build take
 * (exl3_tc_prepare's rules: a hidden size and, at `ranks` ranks, each rank's share of experts.intermediate, split as
 * exl3_output_shard_prepare splits it, in whole blocks the kernels' items cover; routes_per_row and experts_per_layer
 * within the job table's limits). STATUS_UNSUPPORTED with one line naming the model and the first field that does not
 * fit; nothing is printed on success. rotation is accepted for the reference's signature; this build's kernels take
 * any rank's share, so it changes nothing. */
MUST_CHECK result_status exl3_descriptor_tc_check(const char *model_name, const struct exl3_descriptor_model *model, uint32_t ranks,
                                                  uint32_t rotation);

/* The SHA-256 (FIPS 180-4) of `count` bytes; the descriptor's digests are its 64 lower-case hexadecimal digits */
void anemone_sha256(const void *bytes, uint64_t count, unsigned char digest_out[32]);

#ifdef __cplusplus
}
#endif
#endif
