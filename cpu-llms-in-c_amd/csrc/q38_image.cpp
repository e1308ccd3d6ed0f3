// Loader for the four Qwen3.8 image files of the reference's Apple M3 target: a 4096-byte
// header of little-endian scalars, then for each linear a code plane ([rows][cols/2] bytes)
// and a metadata plane ([rows][cols/64] {fp16 scale, fp16 bias}) at the offsets the header
// names (qwen38_m3_image.h:26-87, qwen38_m3_attention_image.h:21-70,
// qwen38_m3_global_image.h:15-44, qwen38_m3_mtp_image.h:16-45; written by
// qwen38_m3_pack.c, validated and mapped by qwen38_m3.m:440-560, qwen38_m3_layer.m:146-200,
// qwen38_m3_attention.m:132-190, qwen38_m3_decode.m:405-470,2360-2380).
// The header is read field by field at fixed byte offsets (the table below; a test compares
// it with offsetof() over the reference's structs), every linear becomes an ordinary prepared
// Q4 weight, and nothing of the model's dimensions is assumed: sizes must be consistent
// with the header's own row and column counts and lie inside the image.
#include "internal.h"

#include <cstdlib>
#include <cstring>
#include <new>

using namespace mi355q;

namespace {

struct Field {
    const char *name;
    uint32_t offset, bytes;
};

// rows / columns of a linear come from header fields; columns either directly or as a
// count of 64-column groups
struct LinearSpec {
    const char *name;
    const char *rows_field, *cols_field;
    bool cols_in_groups;
    const char *prefix;  // "<prefix>_quants_offset", "_quants_bytes", "_metadata_offset", "_metadata_bytes"
    uint32_t min_version;
};

struct Format {
    const char *kind_name;
    unsigned char magic[8];
    uint32_t versions[2];  // accepted (0 = unused)
    const Field *fields;
    size_t field_count;
    const LinearSpec *linears;
    size_t linear_count;
};

#define F(name, offset, bytes) {name, offset, bytes}
const Field kLayerFields[] = {
    F("magic", 0, 8), F("version", 8, 4), F("header_bytes", 12, 4), F("hidden_size", 16, 4), F("rows", 20, 4),
    F("group_size", 24, 4), F("down_rows", 40, 4), F("down_groups_per_row", 44, 4),
    F("gate_quants_offset", 56, 8), F("gate_quants_bytes", 64, 8), F("gate_metadata_offset", 72, 8),
    F("gate_metadata_bytes", 80, 8), F("up_quants_offset", 88, 8), F("up_quants_bytes", 96, 8),
    F("up_metadata_offset", 104, 8), F("up_metadata_bytes", 112, 8), F("down_quants_offset", 120, 8),
    F("down_quants_bytes", 128, 8), F("down_metadata_offset", 136, 8), F("down_metadata_bytes", 144, 8),
    F("layer_index", 284, 4), F("delta_input_rows", 288, 4), F("delta_input_groups_per_row", 292, 4),
    F("delta_output_rows", 296, 4), F("delta_output_groups_per_row", 300, 4),
    F("delta_input_quants_offset", 384, 8), F("delta_input_quants_bytes", 392, 8),
    F("delta_input_metadata_offset", 400, 8), F("delta_input_metadata_bytes", 408, 8),
    F("delta_output_quants_offset", 416, 8), F("delta_output_quants_bytes", 424, 8),
    F("delta_output_metadata_offset", 432, 8), F("delta_output_metadata_bytes", 440, 8)};
const LinearSpec kLayerLinears[] = {
    {"gate", "rows", "hidden_size", false, "gate", 0},
    {"up", "rows", "hidden_size", false, "up", 0},
    {"down", "down_rows", "down_groups_per_row", true, "down", 0},
    // version 2 images hold the MLP only (QWEN38_M3_MLP_ONLY_IMAGE_VERSION)
    {"delta_input", "delta_input_rows", "delta_input_groups_per_row", true, "delta_input", 3},
    {"delta_output", "delta_output_rows", "delta_output_groups_per_row", true, "delta_output", 3}};

const Field kAttentionFields[] = {
    F("magic", 0, 8), F("version", 8, 4), F("header_bytes", 12, 4), F("layer_index", 16, 4),
    F("hidden_size", 20, 4), F("intermediate_size", 24, 4), F("group_size", 28, 4), F("input_rows", 48, 4),
    F("input_groups_per_row", 52, 4), F("output_rows", 56, 4), F("output_groups_per_row", 60, 4),
    F("gate_quants_offset", 72, 8), F("gate_quants_bytes", 80, 8), F("gate_metadata_offset", 88, 8),
    F("gate_metadata_bytes", 96, 8), F("up_quants_offset", 104, 8), F("up_quants_bytes", 112, 8),
    F("up_metadata_offset", 120, 8), F("up_metadata_bytes", 128, 8), F("down_quants_offset", 136, 8),
    F("down_quants_bytes", 144, 8), F("down_metadata_offset", 152, 8), F("down_metadata_bytes", 160, 8),
    F("attention_input_quants_offset", 216, 8), F("attention_input_quants_bytes", 224, 8),
    F("attention_input_metadata_offset", 232, 8), F("attention_input_metadata_bytes", 240, 8),
    F("attention_output_quants_offset", 248, 8), F("attention_output_quants_bytes", 256, 8),
    F("attention_output_metadata_offset", 264, 8), F("attention_output_metadata_bytes", 272, 8)};
const LinearSpec kAttentionLinears[] = {
    {"gate", "intermediate_size", "hidden_size", false, "gate", 0},
    {"up", "intermediate_size", "hidden_size", false, "up", 0},
    {"down", "hidden_size", "intermediate_size", false, "down", 0},
    {"attention_input", "input_rows", "input_groups_per_row", true, "attention_input", 0},
    {"attention_output", "output_rows", "output_groups_per_row", true, "attention_output", 0}};

const Field kGlobalFields[] = {
    F("magic", 0, 8), F("version", 8, 4), F("header_bytes", 12, 4), F("vocab_size", 16, 4),
    F("hidden_size", 20, 4), F("group_size", 24, 4), F("embedding_quants_offset", 40, 8),
    F("embedding_quants_bytes", 48, 8), F("embedding_metadata_offset", 56, 8),
    F("embedding_metadata_bytes", 64, 8), F("lm_head_quants_offset", 72, 8), F("lm_head_quants_bytes", 80, 8),
    F("lm_head_metadata_offset", 88, 8), F("lm_head_metadata_bytes", 96, 8)};
const LinearSpec kGlobalLinears[] = {{"embedding", "vocab_size", "hidden_size", false, "embedding", 0},
                                     {"lm_head", "vocab_size", "hidden_size", false, "lm_head", 0}};

const Field kMtpFields[] = {
    F("magic", 0, 8), F("version", 8, 4), F("header_bytes", 12, 4), F("hidden_size", 16, 4), F("fc_rows", 20, 4),
    F("fc_groups_per_row", 24, 4), F("group_size", 28, 4), F("fc_quants_offset", 40, 8),
    F("fc_quants_bytes", 48, 8), F("fc_metadata_offset", 56, 8), F("fc_metadata_bytes", 64, 8)};
const LinearSpec kMtpLinears[] = {{"fc", "fc_rows", "fc_groups_per_row", true, "fc", 0}};
#undef F

#define COUNT(array) (sizeof(array) / sizeof(array[0]))
const Format kFormats[] = {
    {"layer", {'Q', '3', '8', 'M', '3', 'Q', '4', '\0'}, {3, 2}, kLayerFields, COUNT(kLayerFields), kLayerLinears,
     COUNT(kLayerLinears)},
    {"attention", {'Q', '3', '8', 'M', '3', 'A', 'T', 'T'}, {1, 0}, kAttentionFields, COUNT(kAttentionFields),
     kAttentionLinears, COUNT(kAttentionLinears)},
    {"global", {'Q', '3', '8', 'M', '3', 'G', 'L', 'B'}, {1, 0}, kGlobalFields, COUNT(kGlobalFields),
     kGlobalLinears, COUNT(kGlobalLinears)},
    {"mtp", {'Q', '3', '8', 'M', '3', 'M', 'T', 'P'}, {1, 0}, kMtpFields, COUNT(kMtpFields), kMtpLinears,
     COUNT(kMtpLinears)}};
constexpr size_t kHeaderBytes = 4096;

const Field *find_field(const Format &format, const char *name)
{
    for (size_t i = 0; i < format.field_count; ++i)
        if (strcmp(format.fields[i].name, name) == 0) return &format.fields[i];
    return nullptr;
}

// little-endian scalar of 4 or 8 bytes
bool read_field(const Format &format, const unsigned char *header, const char *name, uint64_t *value)
{
    const Field *field = find_field(format, name);
    if (field == nullptr || (field->bytes != 4 && field->bytes != 8)) return false;
    uint64_t v = 0;
    for (uint32_t b = 0; b < field->bytes; ++b) v |= (uint64_t)header[field->offset + b] << (8 * b);
    *value = v;
    return true;
}

}  // namespace

struct mi355q_q38_image {
    mi355q_context *ctx;
    int kind;
    uint32_t version, layer_index;
    size_t count;
    const char *names[8];
    mi355q_q4_weight *weights[8];
};

extern "C" void mi355q_q38_image_close(mi355q_q38_image *image)
{
    if (image == nullptr) return;
    for (size_t i = 0; i < image->count; ++i) mi355q_q4_weight_destroy(image->weights[i]);
    delete image;
}

extern "C" int mi355q_q38_image_open(mi355q_context *ctx, const void *bytes, size_t size,
                                     mi355q_q38_image **out, char *error, size_t error_capacity)
{
    if (out != nullptr) *out = nullptr;
    if (ctx == nullptr || bytes == nullptr || out == nullptr) {
        set_error(error, error_capacity, "q38_image_open: null argument");
        return MI355Q_ERROR_INVALID;
    }
    const unsigned char *base = (const unsigned char *)bytes;
    if (size < kHeaderBytes) {
        set_error(error, error_capacity, "q38_image_open: %zu bytes is shorter than the %zu-byte header", size,
                  kHeaderBytes);
        return MI355Q_ERROR_INVALID;
    }
    int kind = -1;
    for (size_t f = 0; f < COUNT(kFormats); ++f)
        if (memcmp(base, kFormats[f].magic, 8) == 0) kind = (int)f;
    if (kind < 0) {
        set_error(error, error_capacity, "q38_image_open: unknown magic");
        return MI355Q_ERROR_INVALID;
    }
    const Format &format = kFormats[kind];
    uint64_t version = 0, header_bytes = 0, group_size = 0, layer_index = 0;
    read_field(format, base, "version", &version);
    read_field(format, base, "header_bytes", &header_bytes);
    read_field(format, base, "group_size", &group_size);
    read_field(format, base, "layer_index", &layer_index);  // absent in global / mtp: stays 0
    if ((version != format.versions[0] && (format.versions[1] == 0 || version != format.versions[1])) ||
        header_bytes != kHeaderBytes || group_size != 64) {
        set_error(error, error_capacity,
                  "q38_image_open: %s image with version %llu, header_bytes %llu, group_size %llu", format.kind_name,
                  (unsigned long long)version, (unsigned long long)header_bytes, (unsigned long long)group_size);
        return MI355Q_ERROR_INVALID;
    }
    mi355q_q38_image *image = new (std::nothrow) mi355q_q38_image();
    if (image == nullptr) {
        set_error(error, error_capacity, "q38_image_open: out of host memory");
        return MI355Q_ERROR_RUNTIME;
    }
    memset(image, 0, sizeof *image);
    image->ctx = ctx;
    image->kind = kind;
    image->version = (uint32_t)version;
    image->layer_index = (uint32_t)layer_index;
    for (size_t l = 0; l < format.linear_count; ++l) {
        const LinearSpec &spec = format.linears[l];
        if (version < spec.min_version) continue;
        uint64_t rows = 0, cols = 0, planes[4] = {0, 0, 0, 0};
        static const char *const suffix[4] = {"_quants_offset", "_quants_bytes", "_metadata_offset",
                                              "_metadata_bytes"};
        bool found = read_field(format, base, spec.rows_field, &rows) &&
                     read_field(format, base, spec.cols_field, &cols);
        for (int s = 0; s < 4 && found; ++s) {
            char name[64];
            snprintf(name, sizeof name, "%s%s", spec.prefix, suffix[s]);
            found = read_field(format, base, name, &planes[s]);
        }
        if (spec.cols_in_groups) cols *= 64u;
        const uint64_t code_bytes = rows * cols / 2u, meta_bytes = rows * (cols / 64u) * 4u;
        if (!found || rows == 0 || cols == 0 || cols % 64u != 0 || rows > 0xffffffffull || cols > 0xffffffffull ||
            planes[1] != code_bytes || planes[3] != meta_bytes || planes[0] < kHeaderBytes ||
            planes[2] < kHeaderBytes || planes[0] % 4u != 0 || planes[2] % 4u != 0 || planes[0] > size ||
            code_bytes > size - planes[0] || planes[2] > size || meta_bytes > size - planes[2]) {
            set_error(error, error_capacity,
                      "q38_image_open: %s image, linear %s: %llu x %llu with %llu code bytes at %llu and %llu "
                      "metadata bytes at %llu does not fit the sizes it implies or the image (%zu bytes)",
                      format.kind_name, spec.name, (unsigned long long)rows, (unsigned long long)cols,
                      (unsigned long long)planes[1], (unsigned long long)planes[0], (unsigned long long)planes[3],
                      (unsigned long long)planes[2], size);
            mi355q_q38_image_close(image);
            return MI355Q_ERROR_INVALID;
        }
        mi355q_q4_weight *weight = nullptr;
        int status = mi355q_q4_weight_prepare(ctx, base + planes[0], base + planes[2], nullptr, (uint32_t)rows,
                                              (uint32_t)cols, MI355Q_META_F16_INTERLEAVED, 0, &weight, error,
                                              error_capacity);
        if (status != MI355Q_OK) {
            mi355q_q38_image_close(image);
            return status;
        }
        image->names[image->count] = spec.name;
        image->weights[image->count] = weight;
        ++image->count;
    }
    *out = image;
    return MI355Q_OK;
}

extern "C" int mi355q_q38_image_kind(const mi355q_q38_image *image) { return image ? image->kind : -1; }
extern "C" uint32_t mi355q_q38_image_version(const mi355q_q38_image *image) { return image ? image->version : 0; }
extern "C" uint32_t mi355q_q38_image_layer_index(const mi355q_q38_image *image)
{
    return image ? image->layer_index : 0;
}
extern "C" size_t mi355q_q38_image_linear_count(const mi355q_q38_image *image) { return image ? image->count : 0; }

extern "C" const mi355q_q4_weight *mi355q_q38_image_linear(const mi355q_q38_image *image, size_t index,
                                                          const char **name)
{
    if (image == nullptr || index >= image->count) return nullptr;
    if (name != nullptr) *name = image->names[index];
    return image->weights[index];
}

extern "C" const mi355q_q4_weight *mi355q_q38_image_find(const mi355q_q38_image *image, const char *name)
{
    if (image == nullptr || name == nullptr) return nullptr;
    for (size_t i = 0; i < image->count; ++i)
        if (strcmp(image->names[i], name) == 0) return image->weights[i];
    return nullptr;
}

extern "C" int mi355q_q38_layout_field(int kind, size_t index, const char **name, uint32_t *offset,
                                       uint32_t *bytes)
{
    if (kind < 0 || kind >= (int)COUNT(kFormats) || index >= kFormats[kind].field_count || name == nullptr ||
        offset == nullptr || bytes == nullptr)
        return MI355Q_ERROR_INVALID;
    *name = kFormats[kind].fields[index].name;
    *offset = kFormats[kind].fields[index].offset;
    *bytes = kFormats[kind].fields[index].bytes;
    return MI355Q_OK;
}

extern "C" const char *mi355q_q38_kind_name(int kind)
{
    return kind >= 0 && kind < (int)COUNT(kFormats) ? kFormats[kind].kind_name : nullptr;
}
