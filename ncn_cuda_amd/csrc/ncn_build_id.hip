// The build id of the library: a hash of every source, header and compiler flag it was made from, handed in by the
// build script.  The loader compares it with the hash of the sources it finds, so that a stale library is recognised
// by content whatever the file times say.
#include "../../include/ncn_hip.h"

#ifndef NCN_BUILD_ID_TEXT
#define NCN_BUILD_ID_TEXT "NCN_BUILD_ID=0000000000000000"
#endif

extern "C" const char* ncn_build_id(void) {
    static const char text[] = NCN_BUILD_ID_TEXT;   // "NCN_BUILD_ID=" + 16 hex digits: also found by scanning the file
    return text + sizeof("NCN_BUILD_ID=") - 1;
}
