// Version of the MI355X SCN engine's spconv-compatible C++ surface.
// Counterpart of libraries/3DSparseConvolution/libspconv/include/spconv/version.hpp (API level 1.3.x).
#ifndef SCN_SPCONV_VERSION_HPP
#define SCN_SPCONV_VERSION_HPP

#define NVSPCONV_MAJOR 1
#define NVSPCONV_MINOR 3
#define NVSPCONV_REL 2
#define NVSPCONV_STR(v) #v
#define NVSPCONV_VERSION_COMBIN(major, minor, rel) (NVSPCONV_STR(major) "." NVSPCONV_STR(minor) "." NVSPCONV_STR(rel))
#define NVSPCONV_VERSION NVSPCONV_VERSION_COMBIN(NVSPCONV_MAJOR, NVSPCONV_MINOR, NVSPCONV_REL)
#define SCN_BACKEND "hip-gfx950"

#endif
