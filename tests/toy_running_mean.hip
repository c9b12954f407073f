// A kernel that belongs to a test, not to the library: the mixer of a toy architecture that
// tests/test_gpu_parts.py defines, built as a kernel module of its own ("toy_mean") that the test registers.
//   y[row] = (state[slot] + sum of x over the rows of the same sequence up to and including row) / (position + 1)
//   state[slot] += sum of x over all rows of the sequence
// One thread per (row, channel) for y, one per (sequence, channel) for the state, in that order on the stream.
#include "common.h"

thread_local char g_nnis_error[512] = {0};
extern "C" const char* nnis_last_error() { return g_nnis_error; }

// row_seq: the sequence (index into seq_start / seq_slot) of each row, or a value >= batch for a row that
// belongs to none; null: row r is sequence r (a step of single tokens).
__global__ void toy_mean_rows_kernel(const float* x, const int* row_seq, const int* seq_start, const int* seq_slot,
                                     const int* tok_pos, const float* state, float* y, int rows, int batch, int width) {
  const int index = blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= rows * width) return;
  const int row = index / width, channel = index % width;
  const int seq = row_seq ? row_seq[row] : row;
  const int slot = seq < batch ? seq_slot[seq] : -1;
  if (slot < 0) {
    y[index] = 0.0f;
    return;
  }
  float sum = state[(size_t)slot * width + channel];
  for (int r = seq_start[seq]; r <= row; ++r) sum += x[(size_t)r * width + channel];
  y[index] = sum / (float)(tok_pos[row] + 1);
}

__global__ void toy_mean_state_kernel(const float* x, const int* seq_start, const int* seq_slot, float* state, int batch,
                                      int rows, int width) {
  const int index = blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= batch * width) return;
  const int seq = index / width, channel = index % width;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int first = seq_start[seq], end = min(seq_start[seq + 1], rows);
  float sum = 0.0f;
  for (int r = first; r < end; ++r) sum += x[(size_t)r * width + channel];
  state[(size_t)slot * width + channel] += sum;
}

extern "C" int toy_running_mean(const float* x, const int* row_seq, const int* seq_start, const int* seq_slot, const int* tok_pos,
                                float* state, float* y, int rows, int batch, int width, hipStream_t stream) {
  NNIS_REQUIRE(rows > 0 && batch > 0 && width > 0, "toy_running_mean: sizes must be positive");
  NNIS_REQUIRE(row_seq != nullptr || rows == batch, "toy_running_mean: without a list every row is a sequence");
  hipLaunchKernelGGL(toy_mean_rows_kernel, dim3((rows * width + 255) / 256), dim3(256), 0, stream, x, row_seq, seq_start, seq_slot,
                     tok_pos, state, y, rows, batch, width);
  NNIS_LAUNCH_CHECK("toy_running_mean");
  hipLaunchKernelGGL(toy_mean_state_kernel, dim3((batch * width + 255) / 256), dim3(256), 0, stream, x, seq_start, seq_slot, state,
                     batch, rows, width);
  NNIS_LAUNCH_CHECK("toy_running_mean");
  return 0;
}
