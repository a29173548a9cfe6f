// mock_abi.h -- test hooks of the host mock of the C ABI (mock_abi.cpp).
#pragma once

#include <cstddef>
#include <functional>

#include "mlx_rocm_qmm.h"

// Runs `fn` in `stream`'s order on the mock's stream thread: a stand-in for a
// kernel launch.
void mock_launch(mlxrocm_stream_t stream, std::function<void()> fn);

struct MockCounters {
  long live_device_allocs;
  long live_host_allocs;
  long live_events;
  long live_streams;
  long h2d_copies;
  long d2h_copies;
  long stream_syncs;
};
MockCounters mock_counters();
// Makes the next `n` mlxrocm_event_synchronize calls fail with MLXROCM_HIP_ERROR.
void mock_fail_event_synchronize(int n);
// Makes the next `n` mlxrocm_event_record calls fail with MLXROCM_HIP_ERROR.
void mock_fail_event_record(int n);
// Joins every mock stream thread (after draining it); call at the end of main.
void mock_shutdown();
