/* status.c -- a short English phrase for a status (include/anemone/status.h:37-38 of the reference). */
#include "anemone_backend.h"

const char *status_text(result_status status)
{
    static const char *const phrases[STATUS_COUNT] = {
        [STATUS_OK] = "ok",
        [STATUS_INVALID_ARGUMENT] = "invalid argument",
        [STATUS_OUT_OF_MEMORY] = "out of memory",
        [STATUS_INPUT_OUTPUT_ERROR] = "input/output error",
        [STATUS_CORRUPT_PACK] = "corrupt pack",
        [STATUS_DEVICE_ERROR] = "device error",
        [STATUS_TIMED_OUT] = "timed out",
        [STATUS_UNSUPPORTED] = "unsupported",
        [STATUS_BUSY_VALUE] = "busy",
        [STATUS_INJECTED_FAULT] = "injected fault",
    };
    return (unsigned)status < STATUS_COUNT ? phrases[status] : "unknown status";
}
