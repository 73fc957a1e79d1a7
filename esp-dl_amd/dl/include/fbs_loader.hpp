// Reader for ESP-DL's `.espdl` model containers: header + FlatBuffers payload -> fbs::FbsModel.
//
// Interface after the reference's fbs::FbsLoader (esp-dl/fbs_loader/include/fbs_loader.hpp): construct
// from a location, list / count the models of a package, load one.  Container formats as documented
// there (EDL1 / EDL2 single models, PDL1 / PDL2 packages); the payload follows
// esp-dl/fbs_loader/espdl.fbs and is walked by hand (vtables), with every offset bounds-checked: a
// file is data, nothing in it is executed.
//
// What load() does beyond copying fields:
//   * filters stored for the ESP32-S3 / ESP32-P4 targets in the blocked order the vector units read
//     ("(N/16)HWC16", "N16HWC16", "(N/16)WC16", "(N/8)HWC8", "..._UNALIGNED": blocks of 16 (int8) or
//     8 (int16) filters with the filter index innermost, then the N % block remaining filters in plain
//     filter-major order; depthwise filters are blocked over their channels) are rewritten into the
//     order of the `c` target, [N][H][W][C] (depthwise [H][W][C]), which the kernels here read;
//   * encrypted payloads (mode 1, AES-128) are refused.
#pragma once

#include <string>
#include <vector>

#include "fbs_model.hpp"

namespace fbs {

typedef enum {
    MODEL_LOCATION_IN_FLASH_RODATA = 0, ///< here: a host-memory buffer holding the container
    MODEL_LOCATION_IN_FLASH_PARTITION = 1,
    MODEL_LOCATION_IN_SDCARD = 2, ///< a file path
    MODEL_LOCATION_MAX = MODEL_LOCATION_IN_SDCARD,
} model_location_type_t;

class FbsLoader {
public:
    /// IN_SDCARD: `name` is a file path (read at construction).  The other locations take a pointer to
    /// the container bytes in host memory; use the (data, size) constructor for those, which knows the size.
    FbsLoader(const char *name, model_location_type_t location = MODEL_LOCATION_IN_SDCARD);
    FbsLoader(const void *data, size_t size);
    ~FbsLoader() {}

    /// New FbsModel (caller owns it) or nullptr with the reason in last_error().
    FbsModel *load(const uint8_t *key = nullptr, bool param_copy = true);
    FbsModel *load(int model_index, const uint8_t *key = nullptr, bool param_copy = true);
    FbsModel *load(const char *model_name, const uint8_t *key = nullptr, bool param_copy = true);
    int get_model_num();
    void list_models();
    const char *get_model_location_string();
    const std::string &last_error() const { return m_error; }

private:
    struct Entry {
        std::string name;
        size_t offset; // of the EDLx header inside m_bytes
        int header;    // bytes before the payload: 12 (EDL1) or 16 (EDL2)
    };
    bool index();
    FbsModel *parse(const Entry &e, const uint8_t *key);

    std::vector<uint8_t> m_bytes;
    std::vector<Entry> m_entries;
    model_location_type_t m_location;
    std::string m_error;
    bool m_indexed = false;
};

} // namespace fbs
