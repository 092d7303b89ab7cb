// Paged causal attention on the matrix cores (bfloat16 storage, 32-bit softmax), one
// kernel for prompt portions and for single decoded tokens, plus the merge of split-KV
// partial results.
//
// Work of one wave (a workgroup is one wave of 64 lanes): one segment of the packed
// step (a request's rows), one kv head, 16*NT "rows" and a range of keys.  A row is a
// (token, q head of the kv head's group) pair, row = token * G + head_in_group, so the
// G = nq/nkv q heads that share a kv head share every key and value that is loaded
// (the reference's decode kernel launches one workgroup per q head and reads the keys
// G times: crates/cuda-kernels/tools/tilelang/batch_decode_paged_hd128.py:112-151).
//
// Everything streams from global memory straight into MFMA operands; nothing is staged
// through LDS:
//   S^T[key][row]  = K[key][:] . Q[row][:]      A = K tile (16 keys x 32 d), B = Q (16 rows x 32 d)
//   O^T[d][row]   += V^T[d][key] P^T[key][row]  A = V^T tile (16 d x 32 keys), B = P (16 rows x 32 keys)
// with v_mfma_f32_16x16x32_bf16.  Lane (i = lane%16, g = lane/16) of an operand holds row i and
// 8 contraction elements chosen by g; the result puts element [4g+r][i] into register r of
// lane (i, g).  So after S^T every lane holds, for its own row i, the scores of keys 4g..4g+3
// of each 16-key tile: exactly the 8 keys (two tiles) it must feed as operand B of the second
// product, if the V^T operand lists the keys in the same order.  The value cache is therefore
// laid out [page][kv head][d][slot in page] (d-major), which makes "4 consecutive keys at one d"
// one 8-byte load, as the key cache [page][kv head][slot][d] makes "8 consecutive d of one key"
// one 16-byte load.  Row statistics (running max m, sum l) live in the lanes of their row.
//
// Keys are walked in blocks of 32 aligned to absolute key index.  With splits > 1 the blocks
// of a row range are dealt to `splits` waves, each writing unnormalised float32 partials
// (o, m, l); attn_merge combines them (FlashDecoding, as the reference's split kernels do:
// batch_decode_paged_hd128.py:239-463).  Scores are scaled by scale*log2(e) and exponentiated
// with exp2; probabilities are narrowed to bfloat16 before the second product, as the
// reference does (batch_prefill_paged_hd128.py:219-225); the sum l uses the 32-bit values.
#include "common.h"
#include "attention_static.h"
#include "attention_args.h"
#include "attention_stream.h"
#include "attention_portions.h"
#include "attention_portions_dma.h"

#include <cstdio>
#include <mutex>

namespace arle {

template <int NT>
int launch_attn(const AttnArgs& a, dim3 grid, hipStream_t s) {
  // head_dim 64 and 128 as compile-time values: no test and no branch around a load, so that the keys and
  // values of the next block stay in flight while this block is computed (a load inside a branch makes the
  // next wait a wait for everything)
  if (a.D == 128)
    attn_mfma_kernel<NT, 128, true><<<grid, kWave, 0, s>>>(a);
  else if (a.D == 64)
    attn_mfma_kernel<NT, 64, true><<<grid, kWave, 0, s>>>(a);
  else if (a.D <= 64)
    attn_mfma_kernel<NT, 64, false><<<grid, kWave, 0, s>>>(a);
  else if (a.D <= 128)
    attn_mfma_kernel<NT, 128, false><<<grid, kWave, 0, s>>>(a);
  else
    attn_mfma_kernel<NT, 256, false><<<grid, kWave, 0, s>>>(a);
  return launch_status();
}

inline size_t prefill_lds_bytes(int D) {
  return 2 * (static_cast<size_t>(kPfKeys) * (D + 8) + static_cast<size_t>(D) * (kPfKeys + kPfVPad)) * sizeof(uint16_t);
}

// The list of live (row block, segment) pairs depends on the step, not on the layer: a caller that names the step
// (plan_token != 0, a number that no other step of the process has) gets the planning kernel for the first launch
// of the step only.  What the list was made from is kept here, on the host, and compared.
struct PlanMade {
  long long token = 0;
  const int* seg_row0 = nullptr;
  const int* seg_start = nullptr;
  const int* seg_slot = nullptr;
  unsigned blocks = 0, segments = 0;
  int group = 0, min_rows = 0, listed = 0;
  void* stream = nullptr;
  int device = -1;
};
static PlanMade g_plan_made;

// The list and its counters are one set of device variables a GPU: a list is current only for the stream and the
// device it was made on (another stream's launches are not ordered behind the planning kernel, another device has
// a list of its own), and for the same step, segments and launch shape.
inline bool plan_is_current(const AttnArgs& a, dim3 grid, int min_rows, int listed, hipStream_t s) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) dev = -1;
  const PlanMade now{a.plan_token, a.seg_row0, a.seg_start, a.seg_slot, grid.x, grid.z, a.nq / a.nkv, min_rows, listed,
                     static_cast<void*>(s), dev};
  const bool same = a.plan_token != 0 && dev >= 0 && now.token == g_plan_made.token && now.seg_row0 == g_plan_made.seg_row0 &&
                    now.seg_start == g_plan_made.seg_start && now.seg_slot == g_plan_made.seg_slot &&
                    now.blocks == g_plan_made.blocks && now.segments == g_plan_made.segments &&
                    now.group == g_plan_made.group && now.min_rows == g_plan_made.min_rows && now.listed == g_plan_made.listed &&
                    now.stream == g_plan_made.stream && now.device == g_plan_made.device;
  g_plan_made = now;
  return same;
}

static int g_prefill_pair_up = 1;
static int g_prefill_fixed_rounds = -1;  // items a workgroup up to which they are dealt out before the launch (0: never; -1: by the rule below)
constexpr int kDealtMaxKeys = 4096;      // contexts up to which every launch deals its items out

template <int DMAX, bool EXACT>
int launch_prefill_lds(const AttnArgs& a, dim3 grid, int min_rows, int max_kv_len, hipStream_t s) {
  const size_t lds = prefill_lds_bytes(a.D);
  static size_t allowed = 64 * 1024;  // dynamic LDS above 64 KiB has to be asked for, once per kernel
  if (lds > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_lds_kernel<DMAX, EXACT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (e != hipSuccess) return static_cast<int>(e);
    allowed = lds;
  }
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  const long long items = static_cast<long long>(grid.x) * grid.y * grid.z * a.portion_splits;
  const int per_cu = 1;  // eight waves: two on every SIMD, with all the registers they want
  const unsigned workgroups = static_cast<unsigned>(items < static_cast<long long>(per_cu) * cus ? items : per_cu * cus);
  const int listed = static_cast<long long>(grid.x) * grid.z <= kPfPlanMax && grid.x <= 65535 && grid.z <= 65535;
  if (!plan_is_current(a, grid, min_rows, listed, s))
    attn_prefill_plan_kernel<<<1, 256, 0, s>>>(a.seg_row0, a.seg_start, a.seg_slot, static_cast<int>(grid.z),
                                               static_cast<int>(grid.x), a.nq / a.nkv, min_rows, listed);
  if (a.portion_splits > 1 && !listed) return static_cast<int>(hipErrorInvalidValue);  // the merge walks the list
  // dealt out by the rule of launch_prefill_dma_groups (measured there)
  const int fixed_rounds = g_prefill_fixed_rounds >= 0 ? g_prefill_fixed_rounds : (max_kv_len <= kDealtMaxKeys ? 1 << 20 : 2);
  attn_prefill_lds_kernel<DMAX, EXACT><<<workgroups, kPfWaves * kWave, lds, s>>>(a, min_rows, static_cast<int>(grid.x),
                                                                                static_cast<int>(grid.z), listed, fixed_rounds);
  if (a.portion_splits > 1) {
    const long long most = static_cast<long long>(grid.x) * grid.y * grid.z * (kPfRows / kPfWaves);
    attn_merge_portions_kernel<<<static_cast<unsigned>(most < 4LL * cus ? most : 4LL * cus), kPfWaves * kWave, 0, s>>>(a);
  }
  return launch_status();
}


static int g_prefill_groups = -1;  // -1: the launcher decides; 1, 2: forced (measurements and tests)

template <int GROUPS>
int launch_prefill_dma_groups(const AttnArgs& a, dim3 grid, int min_rows, int cus, int max_kv_len, hipStream_t s) {
  const size_t lds = GROUPS * 2 * kDmStageBytes;
  static bool asked = false;  // dynamic LDS of 64 KiB and more has to be asked for, once
  if (!asked) {
    for (const void* kernel : {reinterpret_cast<const void*>(&attn_prefill_dma_kernel<true, GROUPS>),
                               reinterpret_cast<const void*>(&attn_prefill_dma_kernel<false, GROUPS>)}) {
      hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      if (e != hipSuccess) {
        (void)hipGetLastError();
        return static_cast<int>(e);
      }
    }
    asked = true;
  }
  const long long items = static_cast<long long>(grid.x) * grid.y * grid.z * a.portion_splits;
  const long long places = (GROUPS == 1 ? 2LL : 1LL) * cus;  // two workgroups of four waves a CU, or one of eight
  const unsigned workgroups = static_cast<unsigned>(items < places ? items : places);
  const int listed = static_cast<long long>(grid.x) * grid.z <= kPfPlanMax && grid.x <= 65535 && grid.z <= 65535;
  if (a.portion_splits > 1 && !listed) return static_cast<int>(hipErrorInvalidValue);
  if (!plan_is_current(a, grid, min_rows, listed, s))
    attn_prefill_plan_kernel<<<1, 256, 0, s>>>(a.seg_row0, a.seg_start, a.seg_slot, static_cast<int>(grid.z),
                                               static_cast<int>(grid.x), a.nq / a.nkv, min_rows, listed);
  const int pair_up = GROUPS == 1 && g_prefill_pair_up ? static_cast<int>(cus / (static_cast<long long>(a.nkv) * a.portion_splits)) : 0;
  // Items are dealt out before the launch (see the kernel) when none is long, or when a workgroup gets two at most;
  // with long items, several a workgroup, taking them from the counter follows the compute units' differing speeds
  // and the counter's round trip is little beside an item.  Measured on MI355X, dealt against taken, us: a fresh
  // prompt of 2,048 tokens 56.5 against 65.0, of 1,024 30.7 against 34.9, 504 tokens beside 8 decoded ones 32.9
  // against 42.4, four prompts of 2,048 179 against 190, 512 tokens behind 3,584 cached 62.9 against 71.9, segments
  // of 64 to 800 tokens behind 0 to 2,300 372 against 387; a fresh prompt of 8,192 tokens 615 against 598.
  const int fixed_rounds = g_prefill_fixed_rounds >= 0 ? g_prefill_fixed_rounds : (max_kv_len <= kDealtMaxKeys ? 1 << 20 : 2);
  if (a.P % kDmKeys == 0)
    attn_prefill_dma_kernel<true, GROUPS><<<workgroups, GROUPS * kDmWaves * kWave, lds, s>>>(
        a, min_rows, static_cast<int>(grid.x), static_cast<int>(grid.z), listed, pair_up, fixed_rounds);
  else
    attn_prefill_dma_kernel<false, GROUPS><<<workgroups, GROUPS * kDmWaves * kWave, lds, s>>>(
        a, min_rows, static_cast<int>(grid.x), static_cast<int>(grid.z), listed, pair_up, fixed_rounds);
  if (a.portion_splits > 1) {
    const long long most = static_cast<long long>(grid.x) * grid.y * grid.z * (kPfRows / kPfWaves);
    attn_merge_portions_kernel<<<static_cast<unsigned>(most < 4LL * cus ? most : 4LL * cus), kPfWaves * kWave, 0, s>>>(a);
  }
  return launch_status();
}

int launch_prefill_dma(const AttnArgs& a, dim3 grid, int min_rows, int max_qlen, int max_kv_len, hipStream_t s) {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  // Every row block goes to two groups of waves where workgroups of four waves would leave the chip part empty:
  // with more than one item for every fourth CU and no more than three for every two (two such workgroups fit a
  // CU), or with up to two a CU when the items are unequal (a fresh prompt, whose last rows see all keys and whose
  // first rows few: the launch lasts as long as its heaviest item).  Items of about one length, two a CU, fill the
  // chip best with four waves each.  Measured on MI355X (32 q heads over 8 kv heads, pages of 16), two groups
  // against one: a fresh prompt of 2,048 tokens 60 against 65 us, of 1,024 tokens 31 against 35, 1,024 tokens
  // behind 3,072 cached 87 against 111; but 512 tokens behind 3,584 (keys in four parts) 79 against 68, eight
  // portions of 256 behind 1,024 each 69 against 62, 8,192 fresh tokens 633 against 604; 512 tokens behind 512
  // cached (one item for every second CU) 27 against 33, a fresh prompt of 128 tokens 12.6 against 11.2.
  const long long items = static_cast<long long>(grid.x) * grid.y * grid.z * a.portion_splits;
  const bool unequal = 2LL * max_qlen > max_kv_len;  // the first rows see less than half of what the last see
  const bool two = g_prefill_groups >= 0 ? g_prefill_groups == 2
                                         : (4 * items > cus && (2 * items <= 3LL * cus || (unequal && items <= 2LL * cus)));
  return two ? launch_prefill_dma_groups<2>(a, grid, min_rows, cus, max_kv_len, s)
             : launch_prefill_dma_groups<1>(a, grid, min_rows, cus, max_kv_len, s);
}

// -1: the launcher decides (below); 1: head_dim 128 portions always run attn_prefill_dma_kernel; 0: always
// attn_prefill_lds_kernel, as every other head_dim does.  For measurements and tests that compare the two.
static int g_prefill_dma = -1;

// The kernel with 32 rows a wave does a tile in two thirds of the time.  Measured inside whole prefill steps of the
// Qwen3-4B shape it is level with the other one for a fresh prompt of 512 tokens and 3 to 5 % of the step ahead
// for portions of 512 behind 512 to 3,584 cached tokens, so it takes every portion that it can.
inline bool prefill_dma_pays(dim3 grid, int max_qlen, int max_kv_len) {
  (void)grid;
  (void)max_qlen;
  (void)max_kv_len;
  if (g_prefill_dma >= 0) return g_prefill_dma != 0;
  return true;
}

}  // namespace arle

using namespace arle;

// A mixed step's decoded tokens beside its portions: the two kinds of segments go to kernels of their own that do
// not depend on each other.  With a side branch the split-KV kernel and its merge are queued on a second stream
// (default priority) between an event that forks it off the caller's stream and one that joins it again, so that
// they run beside the portions kernel; a capture of the caller's stream takes the branch in as parallel nodes.
// Measured on MI355X, 8 decoding requests at 2,048 tokens beside a fresh portion of 504 (Qwen3-4B shape): 8.45
// against 8.80 ms a step, the same bits.
static int g_side_branch = 1;
extern "C" void arle_attn_side_branch(int on) { g_side_branch = on; }

namespace {
struct SideBranch {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
};
SideBranch g_side[64];

// the current device's side stream and events, made at the first call outside a capture (nullptr: there is none:
// making a stream while `s` is being captured would break the capture, so such a call does without the branch)
SideBranch* side_branch(hipStream_t s) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  SideBranch& b = g_side[dev];
  if (b.stream == nullptr) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return nullptr;
    }
    if (hipStreamCreateWithFlags(&b.stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&b.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&b.join, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      b = SideBranch{};
      return nullptr;
    }
  }
  return &b;
}
}  // namespace

extern "C" void arle_attn_prefill_variant(int dma) { g_prefill_dma = dma; }
extern "C" void arle_attn_prefill_pair_up(int on) { g_prefill_pair_up = on; }
extern "C" void arle_attn_prefill_fixed_rounds(int rounds) { g_prefill_fixed_rounds = rounds; }
extern "C" void arle_attn_prefill_groups(int groups) { g_prefill_groups = groups; }

// Token rows that the split-KV workspace holds for every segment: the most tokens of a segment whose rows
// (tokens x q heads of a kv head) fit one row tile of 16.
extern "C" int arle_attn_ws_rows(int max_qlen, int nq, int nkv) {
  const int G = nkv > 0 ? nq / nkv : 1;
  return max(1, min(max_qlen, 16 / max(G, 1)));
}

static AttnArgs make_args(const void* q, long long q_stride, void* out, long long o_stride, const void* k_pages,
                          const void* v_pages, const int* block_table, int table_stride, const int* seg_row0,
                          const int* seg_slot, const int* seg_start, int max_qlen, int nq, int nkv, int D,
                          int page_size, float scale, int window, int splits, float* ws_o, float* ws_ml) {
  AttnArgs a;
  a.q = static_cast<const uint16_t*>(q);
  a.q_stride = q_stride;
  a.out = static_cast<uint16_t*>(out);
  a.o_stride = o_stride;
  a.ws_o = ws_o;
  a.ws_ml = ws_ml;
  a.k_pages = static_cast<const uint16_t*>(k_pages);
  a.v_pages = static_cast<const uint16_t*>(v_pages);
  a.block_table = block_table;
  a.table_stride = table_stride;
  a.seg_row0 = seg_row0;
  a.seg_slot = seg_slot;
  a.seg_start = seg_start;
  a.nq = nq;
  a.nkv = nkv;
  a.D = D;
  a.P = page_size;
  a.p_shift = __builtin_ctz(static_cast<unsigned>(page_size));
  a.scale_log2 = scale * 1.4426950408889634f;
  a.window = window;
  a.splits = splits;
  a.ws_rows = arle_attn_ws_rows(max_qlen, nq, nkv);
  a.portion_splits = 1;
  a.plan_token = 0;
  a.pws_o = nullptr;
  a.pws_ml = nullptr;
  a.rows_max = 0;
  a.prep_parts = nullptr;
  a.prep_bf16 = 0;
  a.prep_n = 0;
  a.prep_part_stride = a.prep_row_stride = 0;
  a.prep_qw = a.prep_kw = nullptr;
  a.prep_w_f32 = 0;
  a.prep_cos = a.prep_sin = nullptr;
  a.prep_rot = 0;
  a.prep_eps = 0.f;
  a.prep_k_pages = a.prep_v_pages = nullptr;
  return a;
}

// q, out: bfloat16 [token rows, nq*D] (row strides in elements).  Segments describe the packed
// step: seg_row0[s]..seg_row0[s+1] are the token rows of segment s, whose first token sits at
// position seg_start[s] of the request in block-table row seg_slot[s]; the cache already holds
// the keys and values of these tokens.  max_qlen / min_qlen are the longest and shortest segment, max_kv_len the most
// keys that a segment of more than one token holds after the step (it only steers choices of the portions kernels).  With splits > 1,
// ws_o/ws_ml must hold [segments * ws_rows][nq][splits][D] and [..][2] floats, ws_rows = arle_attn_ws_rows(...),
// and the merge runs after; the split is over the keys of segments of at most 16 rows (decoded tokens and
// portions of a few tokens).  Longer portions go to the LDS kernel; when they have too few row blocks to fill
// the chip, portion_splits > 1 cuts the keys of every row block into that many parts (at most 8), pws_o/pws_ml
// must hold [token rows][nq][portion_splits][D] and [..][2] floats, and a merge of their own runs after.
// plan_token: 0, or a number that names the step (the same for every layer of it, another for every other step of
// the process): the portions kernels then list their work once a step instead of once a call.
// Requires D % 16 == 0, D <= 256, page_size a power of two >= 4.
extern "C" int arle_attn_paged_mfma(const void* q, long long q_stride, void* out, long long o_stride,
                                    const void* k_pages, const void* v_pages, const int* block_table,
                                    int table_stride, const int* seg_row0, const int* seg_slot,
                                    const int* seg_start, int segments, int max_qlen, int min_qlen,
                                    int max_kv_len, int token_rows,
                                    int nq, int nkv, int D, int page_size, float scale, int window,
                                    int splits, float* ws_o, float* ws_ml, int portion_splits, float* pws_o,
                                    float* pws_ml, long long plan_token, void* stream) {
  if (segments == 0 || token_rows == 0) return 0;
  if (D % 16 != 0 || D > 256 || D <= 0 || page_size < 4 || (page_size & (page_size - 1)) != 0 || nq % nkv != 0 ||
      splits < 1 || splits > 64 || portion_splits < 1 || portion_splits > kPortionPartsMax ||
      (portion_splits > 1 && (pws_o == nullptr || pws_ml == nullptr)))
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  AttnArgs a = make_args(q, q_stride, out, o_stride, k_pages, v_pages, block_table, table_stride, seg_row0, seg_slot,
                         seg_start, max_qlen, nq, nkv, D, page_size, scale, window, splits, ws_o, ws_ml);
  a.portion_splits = portion_splits;
  a.pws_o = pws_o;
  a.pws_ml = pws_ml;
  a.plan_token = plan_token;
  const int G = nq / nkv;
  const int max_rows = max_qlen * G, min_rows = min_qlen * G;
  const long long z = static_cast<long long>(segments) * splits;
  if (nkv > 65535 || z > 65535) return static_cast<int>(hipErrorInvalidValue);
  int rc = 0;
  const bool lds_ok = prefill_lds_bytes(D) <= 160 * 1024;
  if (max_rows > 16 && lds_ok) {
    // prompt portions through the LDS kernel; segments of at most 16 rows (decoded tokens of a mixed
    // step) through the streaming kernel
    dim3 grid((max_rows + kPfRows - 1) / kPfRows, nkv, segments);
    SideBranch* side = (min_rows <= 16 && g_side_branch) ? side_branch(s) : nullptr;
    if (side != nullptr) {   // fork: what follows on the side stream waits for what the caller queued so far
      if (hipEventRecord(side->fork, s) != hipSuccess) return static_cast<int>(hipGetLastError());
      if (hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess) {
        side = nullptr;      // nothing was queued on the side stream: go on without the branch
        (void)hipGetLastError();
      }
    }
    int side_rc = 0;
    if (side != nullptr) {
      AttnArgs b = a;
      b.rows_max = 16;
      side_rc = launch_attn<1>(b, dim3(1, nkv, static_cast<unsigned>(z)), side->stream);
      if (side_rc == 0 && splits > 1) {
        attn_merge_kernel<<<dim3(segments * b.ws_rows, nq), kMergeWaves * kWave, 0, side->stream>>>(
            ws_o, ws_ml, b.out, o_stride, seg_row0, b.ws_rows, b.rows_max, nq, nkv, D, splits);
        side_rc = launch_status();
      }
    }
    if (side != nullptr && side_rc != 0) {
      // the branch is forked off already: it is joined before the error goes back, so that a capture of `s` does not
      // end with a stream that never came home, and nothing is still writing when the caller goes on
      if (hipEventRecord(side->join, side->stream) == hipSuccess) (void)hipStreamWaitEvent(s, side->join, 0);
      (void)hipGetLastError();
      return side_rc;
    }
    if (D == 64)
      rc = launch_prefill_lds<64, true>(a, grid, 17, max_kv_len, s);
    else if (D == 128 && page_size % 8 == 0 && static_cast<long long>(nkv) * page_size * D < (1LL << 31) &&
             prefill_dma_pays(grid, max_qlen, max_kv_len))
      rc = launch_prefill_dma(a, grid, 17, max_qlen, max_kv_len, s);
    else if (D == 128)
      rc = launch_prefill_lds<128, true>(a, grid, 17, max_kv_len, s);
    else if (D <= 64)
      rc = launch_prefill_lds<64, false>(a, grid, 17, max_kv_len, s);
    else if (D <= 128)
      rc = launch_prefill_lds<128, false>(a, grid, 17, max_kv_len, s);
    else
      rc = launch_prefill_lds<256, false>(a, grid, 17, max_kv_len, s);
    if (side != nullptr) {   // join: the caller's stream goes on when the side branch is done, also after an error
      const bool joined = hipEventRecord(side->join, side->stream) == hipSuccess && hipStreamWaitEvent(s, side->join, 0) == hipSuccess;
      if (!joined) {
        const int e = static_cast<int>(hipGetLastError());
        return rc != 0 ? rc : e;
      }
      return rc;
    }
    if (rc != 0 || min_rows > 16) return rc;
    a.rows_max = 16;
    rc = launch_attn<1>(a, dim3(1, nkv, static_cast<unsigned>(z)), s);
    if (rc != 0 || splits == 1) return rc;
    attn_merge_kernel<<<dim3(segments * a.ws_rows, nq), kMergeWaves * kWave, 0, s>>>(
        ws_o, ws_ml, a.out, o_stride, seg_row0, a.ws_rows, a.rows_max, nq, nkv, D, splits);
    return launch_status();
  }
  if (max_rows > 16 && splits > 1) return static_cast<int>(hipErrorInvalidValue);  // two row tiles: no split
  // one row tile of 16 when a segment's rows fit it (decoded tokens), else two
  const int nt = max_rows <= 16 ? 1 : 2;
  dim3 grid((max_rows + 16 * nt - 1) / (16 * nt), nkv, static_cast<unsigned>(z));
  rc = nt == 1 ? launch_attn<1>(a, grid, s) : launch_attn<2>(a, grid, s);
  if (rc != 0 || splits == 1) return rc;
  attn_merge_kernel<<<dim3(segments * a.ws_rows, nq), kMergeWaves * kWave, 0, s>>>(
      ws_o, ws_ml, a.out, o_stride, seg_row0, a.ws_rows, 0, nq, nkv, D, splits);
  return launch_status();
}

static int g_decode_inwg = -1;   // the splits of a decode step inside one workgroup: -1 by the rule, 0 never, 1 whenever they fit
extern "C" void arle_attn_decode_inwg(int mode) { g_decode_inwg = mode; }

static int compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  return cus;
}

// A step of single decoded tokens with the preparation of q, k and v folded into the attention: segment s is the
// one token row s.  parts: the fused q|k|v projection of the step as n_parts float32 partial products
// [token rows][(nq + 2 nkv) D] (part_stride elements apart, rows row_stride apart; both multiples of 8, parts
// 16-byte aligned), added in order; or, with parts_bf16, the projection itself in bfloat16 (n_parts 1).  q_w / k_w: per-head norm weights [D] (both or neither; float32 if w_f32, else
// bfloat16; 16-byte aligned), eps inside the root.  cos / sin: float32 [positions][rot / 2], rot 0 (no rotation) or a
// multiple of 64 up to D.  The new token's key and value are written to its slot of the pages (which the block table
// must already hold) and take part in the attention from registers.  D 64 or 128, nq / nkv <= 16; everything else
// as arle_attn_paged_mfma with max_qlen 1.  The same results as arle_qk_prep followed by arle_attn_paged_mfma but
// for the order in which a head's squares are added for its norm.
extern "C" int arle_attn_decode_prep(const void* parts, int parts_bf16, int n_parts, long long part_stride, long long row_stride,
                                     const void* q_w, const void* k_w, int w_f32, const float* cos_t, const float* sin_t,
                                     int rot, float eps, void* out, long long o_stride, void* k_pages, void* v_pages,
                                     const int* block_table, int table_stride, const int* seg_row0, const int* seg_slot,
                                     const int* seg_start, int segments, int nq, int nkv, int D, int page_size,
                                     float scale, int window, int splits, float* ws_o, float* ws_ml, void* stream) {
  if (segments == 0) return 0;
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if ((D != 64 && D != 128) || page_size < 4 || (page_size & (page_size - 1)) != 0 || nkv <= 0 || nq % nkv != 0 ||
      nq / nkv > 16 || splits < 1 || splits > 64 || (splits > 1 && (ws_o == nullptr || ws_ml == nullptr)) ||
      parts == nullptr || n_parts < 1 || (parts_bf16 && n_parts != 1) || part_stride % 8 != 0 || row_stride % 8 != 0 ||
      !aligned(parts) ||
      (q_w == nullptr) != (k_w == nullptr) || !aligned(q_w) || !aligned(k_w) || rot < 0 || rot > D || rot % 64 != 0 ||
      (rot > 0 && (cos_t == nullptr || sin_t == nullptr || !aligned(cos_t) || !aligned(sin_t))) ||
      k_pages == nullptr || v_pages == nullptr || !aligned(k_pages))
    return static_cast<int>(hipErrorInvalidValue);
  const long long z = static_cast<long long>(segments) * splits;
  if (nkv > 65535 || z > 65535) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  AttnArgs a = make_args(nullptr, 0, out, o_stride, k_pages, v_pages, block_table, table_stride, seg_row0, seg_slot,
                         seg_start, 1, nq, nkv, D, page_size, scale, window, splits, ws_o, ws_ml);
  a.prep_parts = parts;
  a.prep_bf16 = parts_bf16;
  a.prep_n = n_parts;
  a.prep_part_stride = part_stride;
  a.prep_row_stride = row_stride;
  a.prep_qw = q_w;
  a.prep_kw = k_w;
  a.prep_w_f32 = w_f32;
  a.prep_cos = cos_t;
  a.prep_sin = sin_t;
  a.prep_rot = rot;
  a.prep_eps = eps;
  a.prep_k_pages = static_cast<uint16_t*>(k_pages);
  a.prep_v_pages = static_cast<uint16_t*>(v_pages);
  // two to four splits and a workgroup for every compute unit even so: the splits of a (segment, kv head) share a
  // workgroup and merge in LDS (measured on MI355X at the Qwen3-4B widths, 64 requests at 2,048 tokens in two splits)
  if (splits > 1 && splits <= kInWgWavesMax && g_decode_inwg != 0 &&
      (g_decode_inwg > 0 || static_cast<long long>(segments) * nkv >= compute_units())) {
    const dim3 grid(1, nkv, static_cast<unsigned>(segments));
    if (D == 128 && parts_bf16)
      attn_mfma_kernel<1, 128, true, true, true, true><<<grid, splits * kWave, 0, s>>>(a);
    else if (D == 128)
      attn_mfma_kernel<1, 128, true, true, true, false><<<grid, splits * kWave, 0, s>>>(a);
    else if (parts_bf16)
      attn_mfma_kernel<1, 64, true, true, true, true><<<grid, splits * kWave, 0, s>>>(a);
    else
      attn_mfma_kernel<1, 64, true, true, true, false><<<grid, splits * kWave, 0, s>>>(a);
    return launch_status();
  }
  const dim3 grid(1, nkv, static_cast<unsigned>(z));
  if (D == 128 && parts_bf16)
    attn_mfma_kernel<1, 128, true, true, false, true><<<grid, kWave, 0, s>>>(a);
  else if (D == 128)
    attn_mfma_kernel<1, 128, true, true, false, false><<<grid, kWave, 0, s>>>(a);
  else if (parts_bf16)
    attn_mfma_kernel<1, 64, true, true, false, true><<<grid, kWave, 0, s>>>(a);
  else
    attn_mfma_kernel<1, 64, true, true, false, false><<<grid, kWave, 0, s>>>(a);
  const int rc = launch_status();
  if (rc != 0 || splits == 1) return rc;
  attn_merge_kernel<<<dim3(segments * a.ws_rows, nq), kMergeWaves * kWave, 0, s>>>(
      ws_o, ws_ml, a.out, o_stride, seg_row0, a.ws_rows, 0, nq, nkv, D, splits);
  return launch_status();
}

// ---- the entry point that allocates nothing (attention_static.h) ---------------------------------------------
//
// The split-KV partial results live in this array.  In host code its name is only a handle for
// hipGetSymbolAddress: each GPU holds its own copy at its own address, looked up once per device below, and
// host code uses that address wherever it needs the memory.
static __device__ __align__(256) float scratch[kAttnStaticOFloats + kAttnStaticMlFloats];

namespace {
constexpr int kStaticDevicesMax = 64;
float* g_static_ptr[kStaticDevicesMax];   // per device: where its copy of `scratch` lies
std::mutex g_static_lock;
thread_local char g_static_error[256] = "";

int static_refuse(const char* what, long long got, long long most) {
  std::snprintf(g_static_error, sizeof(g_static_error), "arle_attn_decode_static: %s %lld exceeds the maximum %lld",
                what, got, most);
  return static_cast<int>(hipErrorInvalidValue);
}

// The current device's address of `scratch` (looked up at the first call on that device, with it current).
int static_scratch(float** ptr) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= kStaticDevicesMax) return static_cast<int>(hipErrorInvalidDevice);
  std::lock_guard<std::mutex> guard(g_static_lock);
  if (g_static_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (p == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
    g_static_ptr[dev] = static_cast<float*>(p);
  }
  *ptr = g_static_ptr[dev];
  return 0;
}
}  // namespace

extern "C" const char* arle_attn_decode_static_error() { return g_static_error; }

extern "C" int arle_attn_decode_static(const void* q, long long q_stride, void* out, long long o_stride,
                                       const void* k_pages, const void* v_pages, const int* block_table,
                                       int table_stride, const int* seg_row0, const int* seg_slot,
                                       const int* seg_start, int segments, int max_qlen, int nq, int nkv, int D,
                                       int page_size, float scale, int window, int splits, void* stream) {
  g_static_error[0] = 0;
  if (segments == 0) return 0;
  if (segments < 0 || max_qlen < 1 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || D % 16 != 0 || D > 256 || D <= 0 ||
      page_size < 4 || (page_size & (page_size - 1)) != 0 || splits < 1 || splits > 64) {
    std::snprintf(g_static_error, sizeof(g_static_error),
                  "arle_attn_decode_static: needs head_dim %% 16 == 0 and <= 256, a power-of-two page size >= 4, "
                  "q heads a multiple of kv heads and 1..64 splits");
    return static_cast<int>(hipErrorInvalidValue);
  }
  const int G = nq / nkv;
  if (static_cast<long long>(max_qlen) * G > 16) return static_refuse("rows of a segment (tokens x group)", static_cast<long long>(max_qlen) * G, 16);
  const long long z = static_cast<long long>(segments) * splits;
  if (nkv > 65535) return static_refuse("kv heads", nkv, 65535);
  if (z > 65535) return static_refuse("segments x splits", z, 65535);
  const long long entries = static_cast<long long>(segments) * arle_attn_ws_rows(max_qlen, nq, nkv) * nq * splits;
  float* ws = nullptr;
  if (splits > 1) {
    if (entries * D > kAttnStaticOFloats) return static_refuse("partial outputs (floats)", entries * D, kAttnStaticOFloats);
    if (entries * 2 > kAttnStaticMlFloats) return static_refuse("partial statistics (floats)", entries * 2, kAttnStaticMlFloats);
    const int rc = static_scratch(&ws);
    if (rc != 0) {
      std::snprintf(g_static_error, sizeof(g_static_error),
                    "arle_attn_decode_static: the device address of the scratch array could not be found (HIP error %d)", rc);
      return rc;
    }
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ws_o = ws;
  float* ws_ml = ws != nullptr ? ws + kAttnStaticOFloats : nullptr;
  AttnArgs a = make_args(q, q_stride, out, o_stride, k_pages, v_pages, block_table, table_stride, seg_row0, seg_slot,
                         seg_start, max_qlen, nq, nkv, D, page_size, scale, window, splits, ws_o, ws_ml);
  int rc = launch_attn<1>(a, dim3(1, nkv, static_cast<unsigned>(z)), s);
  if (rc != 0 || splits == 1) return rc;
  attn_merge_kernel<<<dim3(segments * a.ws_rows, nq), kMergeWaves * kWave, 0, s>>>(
      ws_o, ws_ml, a.out, o_stride, seg_row0, a.ws_rows, 0, nq, nkv, D, splits);
  return launch_status();
}
