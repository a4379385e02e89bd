// Paged decode attention over a hybrid cache for gfx950.
//
// A wavefront owns (sequence, group of HPW adjacent heads, partition): a partition is a run of `partition_size`
// consecutive tokens of one sequence.  Lane layout for a head vector of D elements: LPT = D*elem_bytes/16 lanes
// hold one (token, head) (16 bytes each), the HPW heads of a token sit side by side, so one wave-wide 128-bit
// load covers TPL = 64/(LPT*HPW) tokens; a tile of 16 tokens (never crossing a block because the block size is a
// multiple of 16) takes NG = 16/TPL loads for K and NG for V.  Each of the TPL token rows of the wave runs its
// own online softmax over the tokens it sees (no cross-row traffic in the loop); rows are merged once at the end.
// DEPTH tiles are in flight per wavefront, requested through buffer descriptors so that no load sits under a
// branch.
//
// Per tile the K or V source is chosen per block: block_types[b][i] != 0 reads logical block i from the
// re-projection workspace, otherwise from the persistent K/V cache.
//
// Two ways to put the partitions of a (sequence, head group) together:
//   group path (a sequence has at most 8 partitions): one workgroup per (head group, sequence), wavefront w walks
//     partition w, and the wavefront that finishes last merges the partial results through LDS - one launch, no
//     partial results in HBM.  Workgroups are dealt out longest sequence first.
//   flat path (more partitions than a workgroup has wavefronts): one 64-thread workgroup per (head group,
//     partition, sequence) leaves fp32 partial results and their log-sum-exp; combine_partitions_kernel merges them.
#include <mutex>

#include "paged_decode_core.h"

namespace aps {
namespace {

// seq_order[r] = the sequence with the r-th longest length (ties by index): one thread per sequence.
__global__ __launch_bounds__(256) void rank_sequences_kernel(const int32_t* __restrict__ seq_lens, int batch,
                                                             int32_t* __restrict__ seq_order) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  if (j >= batch) return;
  const int mine = seq_lens[j];
  int rank = 0;
  for (int k = 0; k < batch; ++k) {
    const int other = seq_lens[k];
    rank += (other > mine || (other == mine && k < j)) ? 1 : 0;
  }
  seq_order[rank] = j;
}

// out[b,h,:] = sum_p w_p * part_out[b,h,p,:] / sum_p w_p,  w_p = 2^(lse_p - max lse)
template <int QT>
__global__ __launch_bounds__(256) void combine_partitions_kernel(void* out, const float* part_out,
                                                                const float* part_lse, const int32_t* seq_lens,
                                                                int64_t out_stride, int num_heads, int head_size,
                                                                int num_partitions, int partition_size) {
  const int head = blockIdx.x, seq = blockIdx.y;
  const int seq_len = seq_lens[seq];
  int np = (seq_len + partition_size - 1) / partition_size;
  if (np < 1) np = 1;
  if (np > num_partitions) np = num_partitions;
  const int64_t ph = ((int64_t)seq * num_heads + head) * num_partitions;
  float mx = -INFINITY;
  for (int p = 0; p < np; ++p) mx = fmaxf(mx, part_lse[ph + p]);
  uint16_t* op = (uint16_t*)out + (int64_t)seq * out_stride + (int64_t)head * head_size;
  for (int d = threadIdx.x; d < head_size; d += blockDim.x) {
    float num = 0.f, den = 0.f;
    if (mx != -INFINITY) {
      for (int p = 0; p < np; ++p) {
        const float w = __builtin_amdgcn_exp2f(part_lse[ph + p] - mx);
        num = fmaf(w, part_out[(ph + p) * head_size + d], num);
        den += w;
      }
    }
    op[d] = f32_to_q<QT>(den > 0.f ? num / den : 0.f);
  }
}

inline DecodePlan plan_decode(int64_t batch, int num_heads, int64_t max_seq_len, int partition_size) {
  DecodePlan p{};
  p.np = (max_seq_len + partition_size - 1) / partition_size;
  if (p.np < 1) p.np = 1;
  p.group = p.np <= kMaxGroupWaves;
  p.waves = 1;
  while (p.waves < p.np) p.waves <<= 1;
  // more than one round of resident wavefronts (256 compute units x 16): the order of the workgroups decides
  // how long the last ones run alone
  p.sorted = p.group && batch > 1 && batch * num_heads * p.np > 4096;
  p.order_scratch = p.sorted && batch > kRankInKernelMax;
  return p;
}

template <int QT, int KV, int D, int HPW, int DEPTH>
void launch_group(const AttnArgs& a, int64_t batch, int waves, hipStream_t s) {
  const dim3 grid((unsigned)(a.num_heads / HPW), (unsigned)batch);
  switch (waves) {
    case 1: APS_LAUNCH((paged_decode_group_kernel<QT, KV, D, HPW, DEPTH, 1>), grid, dim3(64), 0, s, a); break;
    case 2: APS_LAUNCH((paged_decode_group_kernel<QT, KV, D, HPW, DEPTH, 2>), grid, dim3(128), 0, s, a); break;
    case 4: APS_LAUNCH((paged_decode_group_kernel<QT, KV, D, HPW, DEPTH, 4>), grid, dim3(256), 0, s, a); break;
    default: APS_LAUNCH((paged_decode_group_kernel<QT, KV, D, HPW, DEPTH, 8>), grid, dim3(512), 0, s, a); break;
  }
}

// Heads per wavefront: adjacent heads of one token are contiguous in memory, so HPW heads per wave make
// the contiguous piece a wave-wide load takes from one token row HPW times longer.
template <int QT, int KV, int D>
void launch_head_size(const AttnArgs& a, int64_t batch, const DecodePlan& plan, hipStream_t s) {
  constexpr int kWant = (KV == KV_FP8) ? APS_HPW_FP8 : APS_HPW_F16;
  constexpr int DEPTH = (KV == KV_FP8) ? APS_DEPTH_FP8 : APS_DEPTH_F16;
  constexpr int LPT = D / Unpack<KV>::EPL;
  constexpr int HPW = (LPT * kWant <= 32) ? kWant : 1;
  if constexpr (HPW > 1) {
    if (a.num_heads % HPW == 0) {
      if (plan.group) {
        launch_group<QT, KV, D, HPW, DEPTH>(a, batch, plan.waves, s);
      } else {
        const dim3 grid((unsigned)(a.num_heads / HPW), (unsigned)a.num_partitions, (unsigned)batch);
        APS_LAUNCH((paged_decode_kernel<QT, KV, D, HPW, DEPTH>), grid, dim3(64), 0, s, a);
      }
      return;
    }
  }
  if (plan.group) {
    launch_group<QT, KV, D, 1, DEPTH>(a, batch, plan.waves, s);
  } else {
    const dim3 grid((unsigned)a.num_heads, (unsigned)a.num_partitions, (unsigned)batch);
    APS_LAUNCH((paged_decode_kernel<QT, KV, D, 1, DEPTH>), grid, dim3(64), 0, s, a);
  }
}

template <int QT, int KV>
int launch_decode(const AttnArgs& a, int head_size, int64_t batch, const DecodePlan& plan, hipStream_t s) {
  if (plan.order_scratch) {
    APS_LAUNCH(rank_sequences_kernel, dim3((unsigned)((batch + 255) / 256)), dim3(256), 0, s, a.seq_lens,
                       (int)batch, const_cast<int32_t*>(a.seq_order));
    const int st = launch_status();
    if (st != APS_OK) return st;
  }
  switch (head_size) {
    case 64: launch_head_size<QT, KV, 64>(a, batch, plan, s); break;
    case 128: launch_head_size<QT, KV, 128>(a, batch, plan, s); break;
    case 256: launch_head_size<QT, KV, 256>(a, batch, plan, s); break;
    case 32:
      if constexpr (KV == KV_FP8) return APS_ERR_UNSUPPORTED;
      else launch_head_size<QT, KV, 32>(a, batch, plan, s);
      break;
    default: return APS_ERR_UNSUPPORTED;
  }
  int st = launch_status();
  if (st != APS_OK || plan.group || a.num_partitions == 1) return st;
  const int threads = head_size >= 256 ? 256 : (head_size + 63) / 64 * 64;
  APS_LAUNCH((combine_partitions_kernel<QT>), dim3((unsigned)a.num_heads, (unsigned)batch), dim3(threads), 0,
                     s, a.out, a.part_out, a.part_lse, a.seq_lens, a.out_stride, a.num_heads, head_size,
                     a.num_partitions, a.partition_size);
  return launch_status();
}

inline int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

}  // namespace
}  // namespace aps

using namespace aps;

extern "C" {

int aps_decode_attention_partition_size(int64_t batch, int num_heads, int64_t max_seq_len, int block_size) {
  if (batch <= 0 || num_heads <= 0 || max_seq_len <= 0 || block_size <= 0) return 256;
  // Aim for a few thousand wavefronts (256 compute units x 8-16 resident waves);
  // shorten the partitions of small batches, never below two tiles.  512 tokens = at most four wavefronts per
  // workgroup for sequences up to 2048: workgroups of four pack the 12 or 16 wave slots of a compute unit
  // without a remainder (8-wavefront workgroups left a third of the slots empty with the fp8 kernel).
  int64_t part = 512;
  while (part > 32 && batch * num_heads * ((max_seq_len + part - 1) / part) < 4096) part >>= 1;
  if (part % block_size != 0) part = (part + block_size - 1) / block_size * block_size;
  // few sequences whose longest still fits the eight wavefronts of one workgroup at partitions of at most 128
  // tokens: take those instead, one launch whose partial results merge in LDS (5 sequences of up to 1000 tokens:
  // 19 against 23-25 us per call; with longer partitions a wavefront walks too many tiles one after the other:
  // one sequence of 2048 tokens, 32 against 23 us)
  if ((max_seq_len + part - 1) / part > kMaxGroupWaves) {
    const int64_t eighth = (max_seq_len + kMaxGroupWaves - 1) / kMaxGroupWaves;
    const int64_t gp = (eighth + block_size - 1) / block_size * block_size;
    if (gp <= 128) part = gp;
  }
  // plenty of sequences: lengthen the partitions until a sequence fits the wavefronts of one workgroup (the
  // partial results then merge in LDS), as far as the 64 block ids a wavefront holds allow
  if (batch * num_heads >= 1024)
    while ((max_seq_len + part - 1) / part > kMaxGroupWaves && 2 * part / block_size <= 64) part *= 2;
  return (int)part;
}

int64_t aps_decode_attention_workspace_bytes(int64_t batch, int num_heads, int head_size, int64_t max_seq_len,
                                             int partition_size) {
  if (batch <= 0 || num_heads <= 0 || head_size <= 0 || max_seq_len <= 0 || partition_size <= 0) return 0;
  const DecodePlan plan = plan_decode(batch, num_heads, max_seq_len, partition_size);
  if (plan.group) return plan.order_scratch ? align_up(batch * 4, 256) : 0;
  const int64_t n = batch * num_heads * plan.np;
  return align_up(n * head_size * 4, 256) + align_up(n * 4, 256);
}

// Checks and plans a call; the scratch for the partial results is the caller's workspace or the library's static
// array.  job.batch == 0 afterwards: nothing to launch.
static int plan_decode_job(PagedJob& job, void* out, const void* q, const void* k_cache, const void* v_cache,
                           const void* ws_k_cache, const void* ws_v_cache, const int32_t* block_tables,
                           const uint8_t* block_types, const int32_t* seq_lens, int64_t batch, int num_heads,
                           int head_size, int block_size, int64_t table_width, int64_t table_stride,
                           int64_t types_stride, int64_t q_stride, int64_t out_stride, int64_t cache_block_stride,
                           int64_t num_cache_blocks, int64_t ws_block_stride, int64_t num_ws_blocks,
                           int64_t max_seq_len, int partition_size, float softmax_scale, int q_dtype, int kv_dtype,
                           float k_scale, float v_scale, void* workspace, int64_t workspace_bytes,
                           int too_small_status) {
  job = PagedJob{};
  job.magic = kPagedJobMagic;
  if (batch < 0 || num_heads <= 0 || head_size <= 0 || block_size <= 0 || table_width < 0) return APS_ERR_INVALID_ARG;
  if (batch == 0) return APS_OK;
  if (!out || !q || !seq_lens) return APS_ERR_INVALID_ARG;
  if (max_seq_len > 0 && (!k_cache || !v_cache || !block_tables)) return APS_ERR_INVALID_ARG;
  if (block_types && (!ws_k_cache || !ws_v_cache)) return APS_ERR_INVALID_ARG;
  if (block_size % kTile != 0) return APS_ERR_UNSUPPORTED;
  if (q_dtype != APS_F16 && q_dtype != APS_BF16) return APS_ERR_UNSUPPORTED;
  if (kv_dtype != q_dtype && kv_dtype != APS_FP8_E4M3) return APS_ERR_UNSUPPORTED;
  if (head_size != 64 && head_size != 128 && head_size != 256 && !(head_size == 32 && kv_dtype != APS_FP8_E4M3))
    return APS_ERR_UNSUPPORTED;   // (the head sizes the kernels are built for: known when a job is planned)
  if (q_stride < (int64_t)num_heads * head_size || out_stride < (int64_t)num_heads * head_size)
    return APS_ERR_INVALID_ARG;
  const int kv_b = kv_dtype == APS_FP8_E4M3 ? 1 : 2;
  const int64_t row = (int64_t)num_heads * head_size;
  if (cache_block_stride < row * block_size || (block_types && ws_block_stride < row * block_size))
    return APS_ERR_INVALID_ARG;
  if (common_vec_bytes({addr(q), addr(out), (uint64_t)q_stride * 2, (uint64_t)out_stride * 2, addr(k_cache),
                        addr(v_cache), addr(ws_k_cache), addr(ws_v_cache), (uint64_t)cache_block_stride * kv_b,
                        (uint64_t)ws_block_stride * kv_b, (uint64_t)head_size * kv_b}) != 16)
    return APS_ERR_UNSUPPORTED;
  if (max_seq_len < 1) max_seq_len = 1;
  if (partition_size <= 0)
    partition_size = aps_decode_attention_partition_size(batch, num_heads, max_seq_len, block_size);
  if (partition_size % block_size != 0 || partition_size / block_size > 64) return APS_ERR_INVALID_ARG;
  const DecodePlan plan = plan_decode(batch, num_heads, max_seq_len, partition_size);
  const int64_t np = plan.np;
  if (np > 65535 || batch > 65535) return APS_ERR_UNSUPPORTED;

  AttnArgs& a = job.a;
  a.out = out;
  a.q = q;
  a.k_cache = (const char*)k_cache; a.v_cache = (const char*)v_cache;
  a.ws_k_cache = (const char*)ws_k_cache; a.ws_v_cache = (const char*)ws_v_cache;
  a.block_tables = block_tables; a.block_types = block_types; a.seq_lens = seq_lens;
  a.q_stride = q_stride; a.out_stride = out_stride; a.table_stride = table_stride; a.types_stride = types_stride;
  a.cache_block_stride_b = cache_block_stride * kv_b; a.ws_block_stride_b = ws_block_stride * kv_b;
  a.num_cache_blocks = num_cache_blocks; a.num_ws_blocks = num_ws_blocks;
  a.num_heads = num_heads; a.block_size = block_size; a.partition_size = partition_size;
  a.num_partitions = (int)np; a.table_width = (int)table_width;
  const float ks = kv_dtype == APS_FP8_E4M3 ? k_scale : 1.f;
  a.scale_log2 = softmax_scale * ks * kLog2e;
  a.v_scale = kv_dtype == APS_FP8_E4M3 ? v_scale : 1.f;
  a.part_out = nullptr; a.part_lse = nullptr; a.seq_order = nullptr;
  a.batch = (int)batch;
  a.rank_in_kernel = plan.sorted && !plan.order_scratch;
  const int64_t need = aps_decode_attention_workspace_bytes(batch, num_heads, head_size, max_seq_len, partition_size);
  if (need > 0) {
    if (workspace && workspace_bytes < need) return too_small_status;
    if (!workspace || (addr(workspace) & 15)) return APS_ERR_WORKSPACE;
    if (plan.group) {
      a.seq_order = (const int32_t*)workspace;
    } else {
      const int64_t n = batch * num_heads * np;
      a.part_out = (float*)workspace;
      a.part_lse = (float*)((char*)workspace + align_up(n * head_size * 4, 256));
    }
  }
  job.head_size = head_size; job.q_dtype = q_dtype; job.kv_dtype = kv_dtype;
  job.plan = plan;
  job.batch = batch;
  return APS_OK;
}

static int launch_decode_job(const PagedJob& job, hipStream_t s) {
  if (job.magic != kPagedJobMagic) return APS_ERR_INVALID_ARG;
  if (job.batch == 0) return APS_OK;
  const bool fp8 = job.kv_dtype == APS_FP8_E4M3;
  if (job.q_dtype == APS_F16) {
    return fp8 ? launch_decode<APS_F16, KV_FP8>(job.a, job.head_size, job.batch, job.plan, s)
               : launch_decode<APS_F16, KV_F16>(job.a, job.head_size, job.batch, job.plan, s);
  }
  return fp8 ? launch_decode<APS_BF16, KV_FP8>(job.a, job.head_size, job.batch, job.plan, s)
             : launch_decode<APS_BF16, KV_BF16>(job.a, job.head_size, job.batch, job.plan, s);
}

int aps_paged_decode_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                               const void* ws_k_cache, const void* ws_v_cache, const int32_t* block_tables,
                               const uint8_t* block_types, const int32_t* seq_lens, int64_t batch, int num_heads,
                               int head_size, int block_size, int64_t table_width, int64_t table_stride,
                               int64_t types_stride, int64_t q_stride, int64_t out_stride,
                               int64_t cache_block_stride, int64_t num_cache_blocks, int64_t ws_block_stride,
                               int64_t num_ws_blocks, int64_t max_seq_len, int partition_size, float softmax_scale,
                               int q_dtype, int kv_dtype, float k_scale, float v_scale, void* workspace,
                               int64_t workspace_bytes, aps_stream_t stream) {
  PagedJob job;
  const int st = plan_decode_job(job, out, q, k_cache, v_cache, ws_k_cache, ws_v_cache, block_tables, block_types, seq_lens,
                                 batch, num_heads, head_size, block_size, table_width, table_stride, types_stride,
                                 q_stride, out_stride, cache_block_stride, num_cache_blocks, ws_block_stride,
                                 num_ws_blocks, max_seq_len, partition_size, softmax_scale, q_dtype, kv_dtype, k_scale,
                                 v_scale, workspace, workspace_bytes, APS_ERR_WORKSPACE);
  return st != APS_OK ? st : launch_decode_job(job, (hipStream_t)stream);
}

int aps_paged_decode_attention_job(void* job, int64_t job_bytes, void* out, const void* q, const void* k_cache,
                                   const void* v_cache, const void* ws_k_cache, const void* ws_v_cache,
                                   const int32_t* block_tables, const uint8_t* block_types, const int32_t* seq_lens,
                                   int64_t batch, int num_heads, int head_size, int block_size, int64_t table_width,
                                   int64_t table_stride, int64_t types_stride, int64_t q_stride, int64_t out_stride,
                                   int64_t cache_block_stride, int64_t num_cache_blocks, int64_t ws_block_stride,
                                   int64_t num_ws_blocks, int64_t max_seq_len, int partition_size,
                                   float softmax_scale, int q_dtype, int kv_dtype, float k_scale, float v_scale,
                                   void* workspace, int64_t workspace_bytes) {
  static_assert(sizeof(PagedJob) <= APS_ATTENTION_JOB_BYTES, "a job fits the bytes the header promises");
  if (!job || job_bytes < (int64_t)sizeof(PagedJob) || (addr(job) & 7)) return APS_ERR_INVALID_ARG;
  return plan_decode_job(*(PagedJob*)job, out, q, k_cache, v_cache, ws_k_cache, ws_v_cache, block_tables, block_types, seq_lens,
                         batch, num_heads, head_size, block_size, table_width, table_stride, types_stride,
                         q_stride, out_stride, cache_block_stride, num_cache_blocks, ws_block_stride,
                         num_ws_blocks, max_seq_len, partition_size, softmax_scale, q_dtype, kv_dtype, k_scale,
                         v_scale, workspace, workspace_bytes, APS_ERR_WORKSPACE);
}

int aps_attention_job_launch(const void* job, aps_stream_t stream) {
  if (!job || (addr(job) & 7)) return APS_ERR_INVALID_ARG;
  return launch_decode_job(*(const PagedJob*)job, (hipStream_t)stream);
}

}  // extern "C"

// ---------------------------------------------------------------- the entry point that allocates nothing
// The partial results of split sequences live in a device array that is part of the library image: every GPU
// the library runs on holds its own copy until the process ends.  In host code the array's name is only a
// handle; the device address is looked up once per device and that pointer is what the kernels receive.
static __device__ __align__(256) unsigned char scratch[APS_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_ptr[kMaxDevices];  // device address of `scratch` on every device seen so far

// Device address of the scratch array on the current device (status != 0: the runtime's error code).
void* scratch_on_current_device(int* status) {
  *status = APS_OK;
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) { *status = (int)e; return nullptr; }
  if (device < 0 || device >= kMaxDevices) { *status = APS_ERR_UNSUPPORTED; return nullptr; }
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[device]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) { *status = e != hipSuccess ? (int)e : APS_ERR_UNSUPPORTED; return nullptr; }
    scratch_ptr[device] = p;
  }
  return scratch_ptr[device];
}
}  // namespace

extern "C" int aps_paged_decode_attention_static(
    void* out, const void* q, const void* k_cache, const void* v_cache, const void* ws_k_cache,
    const void* ws_v_cache, const int32_t* block_tables, const uint8_t* block_types, const int32_t* seq_lens,
    int64_t batch, int num_heads, int head_size, int block_size, int64_t table_width, int64_t table_stride,
    int64_t types_stride, int64_t q_stride, int64_t out_stride, int64_t cache_block_stride, int64_t num_cache_blocks,
    int64_t ws_block_stride, int64_t num_ws_blocks, int64_t max_seq_len, int partition_size, float softmax_scale,
    int q_dtype, int kv_dtype, float k_scale, float v_scale, aps_stream_t stream) {
  int st = APS_OK;
  void* ws = scratch_on_current_device(&st);
  if (st != APS_OK) return st;
  PagedJob job;
  st = plan_decode_job(job, out, q, k_cache, v_cache, ws_k_cache, ws_v_cache, block_tables, block_types, seq_lens,
                       batch, num_heads, head_size, block_size, table_width, table_stride, types_stride,
                       q_stride, out_stride, cache_block_stride, num_cache_blocks, ws_block_stride,
                       num_ws_blocks, max_seq_len, partition_size, softmax_scale, q_dtype, kv_dtype, k_scale,
                       v_scale, ws, APS_STATIC_SCRATCH_BYTES, APS_ERR_SCRATCH_LIMIT);
  return st != APS_OK ? st : launch_decode_job(job, (hipStream_t)stream);
}
