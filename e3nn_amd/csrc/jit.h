// Kernel specialisation helpers (see jit.cpp).
#pragma once
#include <string>

namespace e3x {

// Device template sources, embedded at library build time from templates/*.inc.
extern const char* const kTplCommon;
extern const char* const kTplUvu;
extern const char* const kTplUvuFc;
extern const char* const kTplUvuMfma;
extern const char* const kTplUvwSmall;
extern const char* const kTplUvwMfma;
extern const char* const kTplUvwMfmaBf16;
extern const char* const kTplUvwMfmaDw;
extern const char* const kTplUvwNode;
extern const char* const kTplFcMfma;
extern const char* const kTplFcDw;

std::string cache_dir();

// Returns the path of the code object for `source`, compiling it on a cache miss.
int get_code_object(const std::string& family, const std::string& source, std::string* key_out,
                    std::string* path_out);

}  // namespace e3x
