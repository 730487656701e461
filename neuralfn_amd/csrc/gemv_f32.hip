// Float-activation GEMV / small-batch kernel: one wave per weight row, every
// packed weight decoded once and used for up to R input rows.
//
// This is the exact tier of the library: weights are decoded with the CPU
// engine's arithmetic (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616)
// and multiplied with the float activations as they are; only the order of the
// float additions differs from the engine's double accumulation
// (resident_glimmer.cpp:655-679).  It serves
//   nfn_native_tile_linear_packed_weight_float32_v1 for rows <= 16 and for the
//   encodings without a matrix-core kernel (reference kernel:
//   neuralfn/csrc/tile_cuda/kernels.cu:1398-1525),
//   and the verifier entry points, whose contract is that every row gets the
//   one-row arithmetic (neuralfn/csrc/native_train/tile_ops.h:685-688): the
//   per-row order of operations here does not depend on R.
#include "common.hpp"
#include "gemv_f32_device.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

constexpr int kWavesPerBlock = 4;

template <int R, int P>
__global__ __launch_bounds__(kWavesPerBlock * kWave) void gemv_f32_kernel(
    ProjectionSet set, const float* __restrict__ first, const float* __restrict__ second,
    const float* __restrict__ bias, std::int64_t rows, std::int64_t total_columns) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const std::int64_t column = static_cast<std::int64_t>(blockIdx.x) * kWavesPerBlock + wave;
    if (column >= total_columns) return;
    // Which projection does this column belong to (at most four; uniform per wave).
    int which = 0;
#pragma unroll
    for (int index = 1; index < 4; ++index) {
        if (index < set.count && column >= set.op[index].first_tile) which = index;
    }
    const Projection op = set.op[which];
    const std::int64_t out_col = column - op.first_tile;
    const std::int64_t row0 = static_cast<std::int64_t>(blockIdx.y) * R;
    const int active = static_cast<int>(min(static_cast<std::int64_t>(R), rows - row0));
    const std::int64_t input_dim = set.input_dim;
    const std::uint8_t* row_data = op.data + out_col * op.row_stride;

    float sums[R];
    wave_row_partials<R, P>(op.encoding, row_data, input_dim, first, second, row0, active, lane,
                            sums);

#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float total = wave_sum(sums[r]);
        if (lane == 0 && r < active) {
            op.output[(row0 + r) * op.output_dim + out_col] =
                total + (bias != nullptr ? bias[out_col] : 0.0f);
        }
    }
}

template <int R>
void launch_r(const ProjectionSet& set, const float* first, const float* second, int prologue,
              const float* bias, std::int64_t rows, std::int64_t total_columns,
              hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>((total_columns + kWavesPerBlock - 1) / kWavesPerBlock),
                    static_cast<unsigned>((rows + R - 1) / R), 1);
    const dim3 block(kWavesPerBlock * kWave, 1, 1);
    switch (prologue) {
        case kGated:
            hipLaunchKernelGGL((gemv_f32_kernel<R, kGated>), grid, block, 0, stream, set, first,
                               second, bias, rows, total_columns);
            break;
        case kSwiGlu:
            hipLaunchKernelGGL((gemv_f32_kernel<R, kSwiGlu>), grid, block, 0, stream, set, first,
                               second, bias, rows, total_columns);
            break;
        default:
            hipLaunchKernelGGL((gemv_f32_kernel<R, kPlain>), grid, block, 0, stream, set, first,
                               second, bias, rows, total_columns);
            break;
    }
}

}  // namespace

void launch_gemv_f32(ProjectionSet set, const float* first, const float* second, int prologue,
                     const float* bias, std::int64_t rows, hipStream_t stream) {
    std::int64_t total_columns = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = static_cast<std::uint32_t>(total_columns);
        total_columns += set.op[index].output_dim;
    }
    if (rows == 1) {
        launch_r<1>(set, first, second, prologue, bias, rows, total_columns, stream);
    } else if (rows == 2) {
        launch_r<2>(set, first, second, prologue, bias, rows, total_columns, stream);
    } else if (rows <= 4) {
        launch_r<4>(set, first, second, prologue, bias, rows, total_columns, stream);
    } else {
        launch_r<8>(set, first, second, prologue, bias, rows, total_columns, stream);
    }
}

}  // namespace nfn
