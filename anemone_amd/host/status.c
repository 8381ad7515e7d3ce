/* status.c -- a short English phrase for a status (include/anemone/status.h:37-38 of the reference). */
#include "anemone_backend.h"

const char *status_text(result_status status)
{
    switch (status) {
    case STATUS_OK: return "ok";
    case STATUS_INVALID_ARGUMENT: return "invalid argument";
    case STATUS_OUT_OF_MEMORY: return "out of memory";
    case STATUS_INPUT_OUTPUT_ERROR: return "input/output error";
    case STATUS_CORRUPT_PACK: return "corrupt pack";
    case STATUS_DEVICE_ERROR: return "device error";
    case STATUS_TIMED_OUT: return "timed out";
    case STATUS_UNSUPPORTED: return "unsupported";
    case STATUS_BUSY_VALUE: return "busy";
    case STATUS_INJECTED_FAULT: return "injected fault";
    case STATUS_COUNT: break; /* not a status */
    }
    return "unknown status";
}
