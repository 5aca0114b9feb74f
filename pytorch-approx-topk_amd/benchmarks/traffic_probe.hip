// Memory-traffic probe for the headline shape of the streaming stage-1 kernel.
//
// Issues exactly the loads of stream_kernel<f32, J=2, V=4, W=8, RUN=4> on fp32 x[128, 2^20] with
// 32768 interleaved buckets (a workgroup of 8 waves per 256-column tile, each wave 4 loads of
// 16 bytes per lane, 128 KiB between sub-rows) and then writes 6 KiB per workgroup, the size of
// that kernel's output, in several ways -- with no other work.  The times bound what any kernel
// with this traffic can reach on the machine.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -o traffic_probe traffic_probe.hip && ./traffic_probe
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { \
  std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); std::exit(1); } } while (0)

struct alignas(16) Float4 { float v[4]; };

enum Store { kNone, kStridedOneWave, kDenseOneWave, kDenseAllWaves };

// TILES column tiles per workgroup; a tile is shared by 8 / TILES waves.
template <int TILES, int STORE>
__global__ __launch_bounds__(512) void probe(const float* __restrict__ x, float* __restrict__ out,
                                             int groups_per_row, long long pitch) {
  constexpr int kShare = 8 / TILES, kLoads = 32 / kShare;
  const unsigned lane = threadIdx.x % 64, wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const unsigned group = blockIdx.x % groups_per_row;
  const long long row = blockIdx.x / groups_per_row;
  const unsigned tile = group * TILES + wave / kShare, part = wave % kShare;
  const float* xr = x + row * (pitch * 32) + (long long)tile * 256 + lane * 4;
  Float4 got[kLoads];
#pragma unroll
  for (int u = 0; u < kLoads; ++u) got[u] = *reinterpret_cast<const Float4*>(xr + (long long)(part * kLoads + u) * pitch);
  Float4 best = got[0];
#pragma unroll
  for (int u = 1; u < kLoads; ++u)
#pragma unroll
    for (int e = 0; e < 4; ++e) best.v[e] = fmaxf(best.v[e], got[u].v[e]);
  __shared__ Float4 hand[8][64];
  hand[wave][lane] = best;
  __syncthreads();
  float* o = out + ((long long)blockIdx.x * TILES + wave / kShare) * 1536;  // 6 KiB per tile
  if (STORE == kNone) {
    if (threadIdx.x == 0) out[blockIdx.x] = best.v[0] + hand[7][0].v[1];
  } else if (STORE == kStridedOneWave) {  // two 16-byte stores at 32-byte stride, four at 64-byte stride
    if (part != 0) return;
    *reinterpret_cast<Float4*>(o + lane * 8) = best;
    *reinterpret_cast<Float4*>(o + lane * 8 + 4) = hand[(wave + 1) % 8][lane];
#pragma unroll
    for (int t = 0; t < 4; ++t) *reinterpret_cast<Float4*>(o + 512 + lane * 16 + t * 4) = hand[(wave + 2 + t) % 8][lane];
  } else if (STORE == kDenseOneWave) {    // six stores of 1 KiB
    if (part != 0) return;
#pragma unroll
    for (int t = 0; t < 6; ++t) *reinterpret_cast<Float4*>(o + t * 256 + lane * 4) = hand[(wave + t) % 8][lane];
  } else {                                // every wave of the tile a share of the 6 KiB
    constexpr int kFloats = 1536 / kShare;
    for (int f = lane * 4; f < kFloats; f += 256) *reinterpret_cast<Float4*>(o + part * kFloats + f) = hand[wave][lane];
  }
}

int main() {
  const int rows = 128, inputs = 5;
  const long long pitch = 32768;  // elements between sub-rows
  const size_t n = (size_t)rows * 32 * pitch;
  float* xs[inputs];
  for (int i = 0; i < inputs; ++i) { CHECK(hipMalloc(&xs[i], n * 4)); CHECK(hipMemset(xs[i], i, n * 4)); }
  float* out;
  CHECK(hipMalloc(&out, (size_t)rows * 128 * 6144));
  hipEvent_t start, stop;
  CHECK(hipEventCreate(&start));
  CHECK(hipEventCreate(&stop));
  auto run = [&](const char* name, auto kernel, int tiles_per_group) {
    const int groups = 128 / tiles_per_group;
    for (int i = 0; i < 150; ++i) hipLaunchKernelGGL(kernel, dim3(rows * groups), dim3(512), 0, 0, xs[i % inputs], out, groups, pitch);
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(start));
    const int reps = 300;
    for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(kernel, dim3(rows * groups), dim3(512), 0, 0, xs[i % inputs], out, groups, pitch);
    CHECK(hipEventRecord(stop));
    CHECK(hipEventSynchronize(stop));
    float ms;
    CHECK(hipEventElapsedTime(&ms, start, stop));
    std::printf("%-58s %7.1f us  (%.2f TB/s of reads)\n", name, ms * 1e3 / reps, n * 4 / (ms * 1e-3 / reps) / 1e12);
  };
  run("1 tile per workgroup, 8 waves x 4 loads, no output", probe<1, kNone>, 1);
  run("1 tile, output by one wave, strided (as the product)", probe<1, kStridedOneWave>, 1);
  run("1 tile, output by one wave, dense", probe<1, kDenseOneWave>, 1);
  run("1 tile, output by all waves, dense", probe<1, kDenseAllWaves>, 1);
  run("2 tiles per workgroup, 4 waves x 8 loads, no output", probe<2, kNone>, 2);
  run("2 tiles, output dense", probe<2, kDenseOneWave>, 2);
  run("4 tiles per workgroup, 2 waves x 16 loads, no output", probe<4, kNone>, 4);
  run("4 tiles, output dense", probe<4, kDenseOneWave>, 4);
  run("8 tiles per workgroup, 1 wave x 32 loads, no output", probe<8, kNone>, 8);
  run("8 tiles, output dense", probe<8, kDenseOneWave>, 8);
  return 0;
}
