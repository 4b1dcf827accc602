// Ball query for the local geometric features of GeoTransolver (physicsnemo/nn/module/ball_query.py:32-140 over
// physicsnemo/nn/functional/neighbors/radius_search/_torch_impl.py:59-160, the max_points form): for every query the
// (up to) K nearest points within `radius`, in ascending distance; unused slots hold index 0 and zero coordinates.
//
// One thread per query, 64 queries per workgroup; the points of the query's batch pass through LDS in tiles
// (structure of arrays, read four at a time as wave-wide broadcasts), so the inner loop is vector-ALU work with no
// memory traffic of its own: 3 subtractions, 3 multiply-adds and one comparison per pair.  The rare pair that passes the
// radius test is inserted into the thread's sorted list (distance, index), K entries kept in LDS as [k][thread] so a
// wave's accesses fall on 64 different banks.  Equal distances keep the lower index first.
#include "pa_common.h"
#include "pa_host.h"

namespace pa {
namespace ballquery {

constexpr int kThreads = 64;   // queries per workgroup
constexpr int kTile = 1024;    // points per LDS tile
constexpr int kMaxK = 64;

__global__ __launch_bounds__(kThreads) void ball_query_kernel(const float *__restrict__ points,
                                                              const float *__restrict__ queries, int64_t Np, int64_t Nq,
                                                              int K, float radius, int blocks_per_batch,
                                                              int64_t *__restrict__ indices,
                                                              float *__restrict__ out_points, float *__restrict__ out_dists,
                                                              int32_t *__restrict__ counts) {
  extern __shared__ float lds[];
  float *px = lds;                                  // kTile
  float *py = px + kTile;
  float *pz = py + kTile;
  float *ld = pz + kTile;                           // K * kThreads   distances, ascending
  int *li = reinterpret_cast<int *>(ld + K * kThreads);  // K * kThreads   point indices
  const int t = threadIdx.x;
  const int64_t b = blockIdx.x / blocks_per_batch;
  const int64_t q = (int64_t)(blockIdx.x % blocks_per_batch) * kThreads + t;
  const bool live = q < Nq;
  const float *pb = points + b * Np * 3;
  float qx = 0.f, qy = 0.f, qz = 0.f;
  if (live) {
    const float *qp = queries + (b * Nq + q) * 3;
    qx = qp[0], qy = qp[1], qz = qp[2];
  }
  // a pair is looked at closely when its squared distance is below this bound; the test proper is on the rounded
  // square root, as the reference's is
  const float r2 = radius * radius * 1.00001f + 1e-30f;
  int count = 0;

  auto consider = [&](float dx, float dy, float dz, int j) {
    const float d2 = dx * dx + dy * dy + dz * dz;
    if (d2 <= r2) {
      const float d = sqrtf(d2);
      if (d <= radius && (count < K || d < ld[(K - 1) * kThreads + t])) {
        int pos = count < K ? count : K - 1;
        while (pos > 0 && ld[(pos - 1) * kThreads + t] > d) {
          ld[pos * kThreads + t] = ld[(pos - 1) * kThreads + t];
          li[pos * kThreads + t] = li[(pos - 1) * kThreads + t];
          --pos;
        }
        ld[pos * kThreads + t] = d;
        li[pos * kThreads + t] = j;
        if (count < K) ++count;
      }
    }
  };

  for (int64_t j0 = 0; j0 < Np; j0 += kTile) {
    const int n = (int)min((int64_t)kTile, Np - j0);
    __syncthreads();
    for (int i = t; i < kTile; i += kThreads) {
      // a far-away filler for the tail keeps the inner loop free of bounds tests
      const bool ok = i < n;
      px[i] = ok ? pb[(j0 + i) * 3 + 0] : INFINITY;
      py[i] = ok ? pb[(j0 + i) * 3 + 1] : INFINITY;
      pz[i] = ok ? pb[(j0 + i) * 3 + 2] : INFINITY;
    }
    __syncthreads();
    if (live) {
      const int n4 = (n + 3) & ~3;
      for (int i = 0; i < n4; i += 4) {
        const float4 x4 = *reinterpret_cast<const float4 *>(px + i);
        const float4 y4 = *reinterpret_cast<const float4 *>(py + i);
        const float4 z4 = *reinterpret_cast<const float4 *>(pz + i);
        consider(x4.x - qx, y4.x - qy, z4.x - qz, (int)(j0 + i));
        consider(x4.y - qx, y4.y - qy, z4.y - qz, (int)(j0 + i + 1));
        consider(x4.z - qx, y4.z - qy, z4.z - qz, (int)(j0 + i + 2));
        consider(x4.w - qx, y4.w - qy, z4.w - qz, (int)(j0 + i + 3));
      }
    }
  }
  if (!live) return;
  const int64_t row = b * Nq + q;
  for (int k = 0; k < K; ++k) {
    const bool used = k < count;
    const int j = used ? li[k * kThreads + t] : 0;
    indices[row * K + k] = j;
    if (out_points) {
      float *o = out_points + (row * K + k) * 3;
      o[0] = used ? pb[(int64_t)j * 3 + 0] : 0.f;
      o[1] = used ? pb[(int64_t)j * 3 + 1] : 0.f;
      o[2] = used ? pb[(int64_t)j * 3 + 2] : 0.f;
    }
    if (out_dists) out_dists[row * K + k] = used ? ld[k * kThreads + t] : 0.f;
  }
  if (counts) counts[row] = count;
}

// ------------------------------------------------------------------------------------------------
// ball_query_cells_kernel: the same search over a cell list, for clouds where looking at every pair costs too much.
// The caller has binned the points of every batch into G^3 cells of edge >= radius (per axis: origin and 1 / edge in
// `grid` (B, 6)), sorted them by cell (cell index (ix * G + iy) * G + iz) and given the offsets of every cell in the
// sorted order (`cell_start`, B * G^3 + 1 entries, offsets into the flattened (B * Np) sorted arrays).  A query looks
// at the 3 x 3 columns of cells around its own; the three cells of a column are adjacent in the sorted order, so that
// is nine contiguous runs of candidates.  `query_order` (optional) lists the queries of each batch in an order that
// keeps neighbours in space in neighbouring lanes, so that a wave reads the same runs.
// Candidates arrive in cell order, not index order: equal distances are ordered by index explicitly.
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void ball_query_cells_kernel(
    const float *__restrict__ grid, const float *__restrict__ sorted_points, const int32_t *__restrict__ sorted_index,
    const int32_t *__restrict__ cell_start, const float *__restrict__ queries, const int32_t *__restrict__ query_order,
    int64_t Nq, int G, int K, float radius, int blocks_per_batch, int64_t *__restrict__ indices,
    float *__restrict__ out_points, float *__restrict__ out_dists, int32_t *__restrict__ counts) {
  extern __shared__ float lds[];
  float *ld = lds;                                        // K * kThreads
  int *li = reinterpret_cast<int *>(ld + K * kThreads);   // K * kThreads  positions in the sorted order
  const int t = threadIdx.x;
  const int64_t b = blockIdx.x / blocks_per_batch;
  const int64_t slot = (int64_t)(blockIdx.x % blocks_per_batch) * kThreads + t;
  if (slot >= Nq) return;
  const int64_t q = query_order ? query_order[b * Nq + slot] : slot;
  const float *qp = queries + (b * Nq + q) * 3;
  const float qx = qp[0], qy = qp[1], qz = qp[2];
  const float *gr = grid + b * 6;
  // cell coordinates of the query, not clamped to the grid (a query outside the box still sees the border cells)
  const float lim = (float)(G + 1);
  const int cx = (int)floorf(fminf(fmaxf((qx - gr[0]) * gr[3], -2.f), lim));
  const int cy = (int)floorf(fminf(fmaxf((qy - gr[1]) * gr[4], -2.f), lim));
  const int cz = (int)floorf(fminf(fmaxf((qz - gr[2]) * gr[5], -2.f), lim));
  const float r2 = radius * radius * 1.00001f + 1e-30f;
  const int32_t *cs = cell_start + b * (int64_t)G * G * G;
  int count = 0;
  const int z0 = max(cz - 1, 0), z1 = min(cz + 1, G - 1);
  if (z0 <= z1) {
    for (int ix = max(cx - 1, 0); ix <= min(cx + 1, G - 1); ++ix)
      for (int iy = max(cy - 1, 0); iy <= min(cy + 1, G - 1); ++iy) {
        const int64_t column = ((int64_t)ix * G + iy) * G;
        const int begin = cs[column + z0], end = cs[column + z1 + 1];
        for (int j = begin; j < end; ++j) {
          const float dx = sorted_points[(int64_t)j * 3 + 0] - qx;
          const float dy = sorted_points[(int64_t)j * 3 + 1] - qy;
          const float dz = sorted_points[(int64_t)j * 3 + 2] - qz;
          const float d2 = dx * dx + dy * dy + dz * dz;
          if (d2 > r2) continue;
          const float d = sqrtf(d2);
          if (d > radius) continue;
          const int id = sorted_index[j];
          if (count == K) {
            const float worst = ld[(K - 1) * kThreads + t];
            if (d > worst || (d == worst && id > sorted_index[li[(K - 1) * kThreads + t]])) continue;
          }
          int pos = count < K ? count : K - 1;
          while (pos > 0) {
            const float dp = ld[(pos - 1) * kThreads + t];
            if (dp < d || (dp == d && sorted_index[li[(pos - 1) * kThreads + t]] < id)) break;
            ld[pos * kThreads + t] = dp;
            li[pos * kThreads + t] = li[(pos - 1) * kThreads + t];
            --pos;
          }
          ld[pos * kThreads + t] = d;
          li[pos * kThreads + t] = j;
          if (count < K) ++count;
        }
      }
  }
  const int64_t row = b * Nq + q;
  for (int k = 0; k < K; ++k) {
    const bool used = k < count;
    const int j = used ? li[k * kThreads + t] : 0;
    indices[row * K + k] = used ? sorted_index[j] : 0;
    if (out_points) {
      float *o = out_points + (row * K + k) * 3;
      o[0] = used ? sorted_points[(int64_t)j * 3 + 0] : 0.f;
      o[1] = used ? sorted_points[(int64_t)j * 3 + 1] : 0.f;
      o[2] = used ? sorted_points[(int64_t)j * 3 + 2] : 0.f;
    }
    if (out_dists) out_dists[row * K + k] = used ? ld[k * kThreads + t] : 0.f;
  }
  if (counts) counts[row] = count;
}

int ball_query_cells(int64_t B, int64_t Np, int64_t Nq, int64_t K, float radius, int64_t G, const float *grid,
                     const float *sorted_points, const int32_t *sorted_index, const int32_t *cell_start,
                     const float *queries, const int32_t *query_order, int64_t *indices, float *out_points,
                     float *out_dists, int32_t *counts, hipStream_t st) {
  if (K < 1 || K > kMaxK || G < 1 || G > 256 || B * Np > INT32_MAX || B * G * G * G > INT32_MAX) return PA_ERR_UNSUPPORTED;
  const int64_t per_batch = (Nq + kThreads - 1) / kThreads;
  if (B * per_batch > INT32_MAX) return PA_ERR_UNSUPPORTED;
  const size_t lds = 2 * (size_t)K * kThreads * sizeof(float);
  hipLaunchKernelGGL(ball_query_cells_kernel, dim3((unsigned)(B * per_batch)), dim3(kThreads), lds, st, grid,
                     sorted_points, sorted_index, cell_start, queries, query_order, Nq, (int)G, (int)K, radius,
                     (int)per_batch, indices, out_points, out_dists, counts);
  return launch_status();
}

int ball_query(int64_t B, int64_t Np, int64_t Nq, int64_t K, float radius, const float *points, const float *queries,
               int64_t *indices, float *out_points, float *out_dists, int32_t *counts, hipStream_t st) {
  if (K < 1 || K > kMaxK || Np > INT32_MAX) return PA_ERR_UNSUPPORTED;
  const int64_t per_batch = (Nq + kThreads - 1) / kThreads;
  if (B * per_batch > INT32_MAX) return PA_ERR_UNSUPPORTED;
  const size_t lds = (3 * kTile + 2 * (size_t)K * kThreads) * sizeof(float);
  hipLaunchKernelGGL(ball_query_kernel, dim3((unsigned)(B * per_batch)), dim3(kThreads), lds, st, points, queries, Np, Nq,
                     (int)K, radius, (int)per_batch, indices, out_points, out_dists, counts);
  return launch_status();
}

}  // namespace ballquery
}  // namespace pa
