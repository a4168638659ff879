// C interface of the cache manager (cache_manager.cpp), for the other files of the host library.
#pragma once
#include <cstdint>

extern "C" {
int cm_add_request(void* h, int64_t id);
int cm_can_reserve(void* h, int64_t id, int64_t new_len);
int cm_fits_at_all(void* h, int64_t new_len);
int cm_can_admit(void* h, int64_t total_len, int64_t first_len);
int cm_has_window(void* h);
int cm_reserve(void* h, int64_t id, int64_t new_len);
int cm_free(void* h, int64_t id);
int cm_num_free_slots(void* h);
int cm_num_requests(void* h);
int cm_state_slot(void* h, int64_t id);
}
