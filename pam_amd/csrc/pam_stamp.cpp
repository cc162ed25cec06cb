// The hash of the sources this library was built from (pam_amd/build.py passes it in).  It lives in a
// translation unit of its own so that stamping costs no recompilation of the kernels, and behind a tag
// so that a build script can read it from the file's bytes without loading the library.
#ifndef PAM_HIP_SOURCE_HASH
#define PAM_HIP_SOURCE_HASH "unstamped"
#endif

namespace {
const char kStamp[] = "pam_hip_source_hash=" PAM_HIP_SOURCE_HASH;
}

extern "C" const char* pam_hip_source_hash(void) { return kStamp + sizeof("pam_hip_source_hash=") - 1; }
