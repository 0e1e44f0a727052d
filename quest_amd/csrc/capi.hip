// Version and status text of libquest_hip.
#include "common.h"

extern "C" int quest_version(void) { return 101; }

extern "C" const char *quest_status_string(int status) {
    switch (status) {
        case QUEST_OK: return "ok";
        case QUEST_ERR_NULL_POINTER: return "a required pointer is NULL";
        case QUEST_ERR_BAD_SHAPE: return "bad shape (non-positive size, or K not a multiple of what the kernel needs)";
        case QUEST_ERR_BAD_DTYPE: return "dtype is neither bfloat16 (0) nor float16 (1)";
        case QUEST_ERR_ALIGNMENT: return "a pointer is not aligned for the vector accesses used";
        case QUEST_ERR_UNSUPPORTED: return "shape outside what this build instantiates";
        case QUEST_ERR_LAUNCH: return "the HIP runtime reported an error for the launch";
        default: return "unknown status";
    }
}
