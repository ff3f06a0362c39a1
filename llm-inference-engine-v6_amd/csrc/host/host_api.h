// Codes shared by the host runtime's C interface (the cache manager and the scheduler) and
// their Python faces. Calls return a value >= 0 on success and one of these on failure.
#pragma once

enum LlmeHostCode : int {
    LLME_HOST_ALREADY_LIVE = -1,
    LLME_HOST_NO_SLOT = -2,
    LLME_HOST_NOT_LIVE = -3,
    LLME_HOST_NOT_RESERVED = -4,
    LLME_HOST_NOT_HELD = -5,
    LLME_HOST_BAD_ARGUMENT = -6,
    LLME_HOST_CHECK_PAGE_TWICE = -10,
    LLME_HOST_CHECK_PAGE_MISMATCH = -11,
    LLME_HOST_CHECK_PAGE_LOST = -12,
    LLME_HOST_CHECK_SLOT_TWICE = -13,
    LLME_HOST_CHECK_SLOT_LOST = -14,
};
