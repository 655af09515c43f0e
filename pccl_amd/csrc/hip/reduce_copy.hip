// reduce_copy.hip -- pccl_hip_reduce_copy: argument checks, alignment analysis,
// launch shape, dispatch to the typed kernels.
#include <algorithm>
#include <cstring>

#include "reduce_copy_kernel.h"

namespace pccl_dev {

int launch_copy(int elem_bytes, int unroll, bool aligned, int mem, unsigned grid, unsigned lds,
                hipStream_t stream, const RcLaunch &p) {
  // the dtype only selects the element size and the alignment the unaligned pack type may assume
  if (elem_bytes == 8) return launch_nin<PCCL_F64, OpSum, 1>(unroll, aligned, mem, grid, lds, stream, p);
  if (elem_bytes == 4) return launch_nin<PCCL_F32, OpSum, 1>(unroll, aligned, mem, grid, lds, stream, p);
  if (elem_bytes == 2) return launch_nin<PCCL_BF16, OpSum, 1>(unroll, aligned, mem, grid, lds, stream, p);
  return launch_nin<PCCL_F8E4M3, OpSum, 1>(unroll, aligned, mem, grid, lds, stream, p);
}

}  // namespace pccl_dev

using namespace pccl_dev;
using pccl_host::fail;

namespace pccl_host {

// Shared with the graph builder: validates one op's operands and fills the
// launch record.  Returns PCCL_OK or an error code (text set).
int plan_reduce_copy(int dtype, int compute, const void *const *ins, int n_in, void *const *outs,
                     int n_out, long count, RcLaunch *out, bool *aligned) {
  if (dtype < 0 || dtype >= PCCL_NUM_DTYPES) return fail(PCCL_ERR_UNSUPPORTED, "unknown dtype code %d", dtype);
  if (compute < PCCL_SUM || compute > PCCL_MAX)
    return fail(PCCL_ERR_UNSUPPORTED, "unknown compute code %d", compute);
  if (n_in < 1 || n_in > PCCL_MAX_INPUTS) return fail(PCCL_ERR_INVALID_ARG, "n_in %d outside [1, 8]", n_in);
  if (n_out < 1 || n_out > PCCL_MAX_OUTPUTS) return fail(PCCL_ERR_INVALID_ARG, "n_out %d outside [1, 8]", n_out);
  if (count < 0) return fail(PCCL_ERR_INVALID_ARG, "count %ld < 0", count);
  if (!ins || !outs) return fail(PCCL_ERR_INVALID_ARG, "operand array is null");
  const int es = pccl_host::pccl_dtype_bytes(dtype);
  RcLaunch p;
  memset(&p, 0, sizeof(p));
  for (int k = 0; k < n_in; ++k) {
    if (!ins[k] && count) return fail(PCCL_ERR_INVALID_ARG, "input %d is null", k);
    if ((uintptr_t)ins[k] % es) return fail(PCCL_ERR_MISALIGNED, "input %d (%p) not %d-byte aligned", k, ins[k], es);
    p.ops.in[k] = (const char *)ins[k];
  }
  for (int j = 0; j < n_out; ++j) {
    if (!outs[j] && count) return fail(PCCL_ERR_INVALID_ARG, "output %d is null", j);
    if ((uintptr_t)outs[j] % es) return fail(PCCL_ERR_MISALIGNED, "output %d (%p) not %d-byte aligned", j, outs[j], es);
    p.ops.out[j] = (char *)outs[j];
  }
  p.ops.n_out = n_out;
  p.count = count;
  // peel a head so that output 0 starts its body on a 16-byte boundary
  long head = (long)((16 - ((uintptr_t)outs[0] & 15)) & 15) / es;
  if (head > count) head = count;
  p.head = head;
  p.n_packs = (count - head) / (16 / es);
  bool al = true;  // do all other streams land on 16 bytes after the same peel?
  for (int k = 0; k < n_in; ++k) al = al && (((uintptr_t)ins[k] + (uintptr_t)head * es) & 15) == 0;
  for (int j = 0; j < n_out; ++j) al = al && (((uintptr_t)outs[j] + (uintptr_t)head * es) & 15) == 0;
  *aligned = al;
  *out = p;
  return PCCL_OK;
}

}  // namespace pccl_host

extern "C" int pccl_hip_reduce_copy(int dtype, int compute, const void *const *ins, int n_in,
                                    void *const *outs, int n_out, long count, void *stream) {
  pccl_host::clear_error();
  RcLaunch p;
  bool aligned = false;
  int rc = pccl_host::plan_reduce_copy(dtype, compute, ins, n_in, outs, n_out, count, &p, &aligned);
  if (rc != PCCL_OK) return rc;
  if (count == 0) return PCCL_OK;
  const pccl_host::Tuning t = pccl_host::tuning();
  const int es = pccl_host::pccl_dtype_bytes(dtype);
  // A grid times its 256 lanes must fit 32 bits: 2^24 - 1 workgroups of 4 KiB each, just under 64 GiB
  // per stream.  Longer operands run as launches over consecutive slices of 32 GiB (a multiple of
  // 4 KiB: every slice has the alignment of the whole, and the same launch shape).
  const long slice = pccl_host::slice_bytes() / es;
  if (count > slice) {
    for (long lo = 0; lo < count; lo += slice) {
      const void *in_at[PCCL_MAX_INPUTS];
      void *out_at[PCCL_MAX_OUTPUTS];
      for (int k = 0; k < n_in; ++k) in_at[k] = (const char *)ins[k] + lo * es;
      for (int j = 0; j < n_out; ++j) out_at[j] = (char *)outs[j] + lo * es;
      rc = pccl_hip_reduce_copy(dtype, compute, in_at, n_in, out_at, n_out, std::min(slice, count - lo), stream);
      if (rc != PCCL_OK) return rc;
    }
    return PCCL_OK;
  }
  // Operands that together exceed what the 256 MB Infinity Cache can hold run one
  // pack per lane under an occupancy cap (below).  Streaming treatment starts earlier,
  // at 48 MiB: a collective step works on data that just arrived and will not be
  // touched again soon; smaller operands stay cacheable.  Which streaming treatment
  // (measured on MI355X, TB/s with non-temporal stores vs write-through stores):
  //  - same buffers every launch: 8 -> 1 at 256 MiB 6.5 vs 6.6, 8 -> 2 at 128 MiB 6.5 vs
  //    6.9, 4 -> 1 6.3 vs 6.7, 2 -> 1 6.6 vs 7.2;
  //  - walks over distinct buffers (nothing in any cache): copy 1 -> 1 at 96 MiB .. 1 GiB
  //    6.0-6.4 vs 6.3-6.7, 1 -> 2 6.1 vs 6.3, but 1 -> 4 and 1 -> 8 6.6 vs 6.0-6.3;
  //  - a walk over 14 ring steps (7 reductions 2 -> 2, 7 copies): 243 vs 229 us at 32 MiB
  //    chunks, 452 vs 433 us at 64 MiB, when every step uses the same treatment; MIXING
  //    them is worse than either (write-through reductions followed by non-temporal
  //    copies: 249 and 467 us), which is why one rule covers reductions and copies;
  //  - reductions of three and more inputs over several GiB: i32 4 -> 1 at 1 GiB per operand 6.1 vs
  //    6.0, unaligned 5.9 vs 5.4; bf16 4 -> 1 at 4 / 8 / 32 GiB per operand 6.25 / 6.31 / 6.17 vs 6.18 /
  //    6.21 / 6.13.  Copies and 2 -> 1 of that size stay with write-through stores: copy at 4 .. 32 GiB
  //    6.3 vs 6.6, 2 -> 1 6.26-6.46 vs 6.30-6.55.
  const long total_bytes = (long)(n_in + n_out) * count * es;
  const bool big = total_bytes > (192l << 20);
  int mem = kLaunchMemCached;
  if (total_bytes >= (48l << 20)) {
    // (three and four inputs already from 1.4 GiB in all, i32, three allocations each, write-through vs
    // non-temporal: 4 -> 1 at 256 MiB per operand 6.82 vs 6.56 but at 320 MiB 6.44 vs 6.58, 384 MiB 6.47 vs
    // 6.66, 512 MiB 6.44 vs 6.63, 768 MiB 6.51 vs 6.57; 3 -> 1 at 256 MiB 7.27 vs 6.73 but at 384 MiB 6.59 vs
    // 6.75, 512 MiB 6.56 vs 6.65, 1 GiB 6.46 vs 6.56; five to eight inputs keep write-through stores up
    // to 4 GiB: 5 -> 1 at 320 MiB 6.68 vs 6.62, 7 -> 1 at 384 MiB 6.75 vs 6.75, 8 -> 1 at 256 MiB 6.86 vs 6.56)
    const bool few_inputs_large = (n_in == 3 || n_in == 4) && n_out == 1 && total_bytes >= (1408l << 20);
    const bool non_temporal_stores = (n_in == 1 && n_out >= 3) || few_inputs_large || (n_in >= 3 && total_bytes > (4l << 30));
    mem = non_temporal_stores ? kLaunchMemStream : kLaunchMemStreamWriteThrough;
  }
  if (t.cache_treatment >= 0) mem = std::min(t.cache_treatment, (int)kLaunchMemStreamWriteThrough);
  // one pack per lane beyond the Infinity Cache; a copy already from 32 MiB in all (cold walk
  // over 16 MiB copies: 4.55 vs 4.29 TB/s, 64 MiB: 5.8 vs 5.7)
  int unroll = (big || (n_in == 1 && total_bytes >= (32l << 20))) ? 1 : small_unroll_for(n_in);
  if (t.unroll == 1 || t.unroll == 4) unroll = t.unroll == 4 ? small_unroll_for(n_in) : 1;
  // lean kernel wherever nothing has to be peeled and there are at most two outputs.  Kernel
  // durations by rocprofv3, 4 packs per lane in the general kernel vs lean: f32 2 -> 1 at 64 KiB
  // per buffer 2.60 vs 2.36 us, 256 KiB 2.88 vs 2.16, 1 MiB 3.16 vs 2.52, 4 MiB 3.44 vs 2.92,
  // 8 MiB 4.52 vs 3.88; 2 -> 2 at 2 MiB 3.40 vs 2.72; copy of 512 KiB 2.92 vs 2.36, of 3 MiB
  // 2.96 vs 2.56; back-to-back launches on the same buffers, 2 -> 1 and 2 -> 2 at 8 .. 32 MiB per
  // buffer: +4 .. +11 % (2 -> 2 at 32 MiB: -2 %), everything else within 1 %.
  const int epp = 16 / es;
  const bool lean_ok = aligned && p.head == 0 && p.n_packs * epp == count && n_out <= 2 && t.workgroups_per_cu == 0;
  if (lean_ok && t.unroll <= 0) unroll = 0;
  const long chunk = (long)kBlock * (unroll ? unroll : 1);
  long chunks = (p.n_packs + chunk - 1) / chunk;
  if (chunks < 1) chunks = 1;
  // default: one workgroup per chunk; a tuning run may cap it to a persistent grid
  long grid = chunks;
  if (t.workgroups_per_cu > 0) grid = std::min<long>(chunks, (long)pccl_host::compute_units() * t.workgroups_per_cu);
  // (the general kernel's chunk loop covers whatever a clamped grid leaves; the lean kernel has no
  // loop and sizes its own grid in launch_lean_nout, one workgroup per 4 KiB: 2^31 of them are 8 TiB
  // per stream, more than the device holds)
  if (grid > 0x7fffffffl) grid = 0x7fffffffl;
  // Occupancy cap for operands beyond the Infinity Cache.  Measured on MI355X: DRAM
  // efficiency is best with about 20 (workgroups x streams) resident per compute
  // unit, i.e. 2 workgroups for 8 -> 1 (+8 %), 5 for 2 -> 2 (+10 %), no cap for a
  // copy; more concurrent streams per memory channel cost row-buffer locality.  The
  // cap is imposed by requesting dynamic LDS the kernel never touches.
  unsigned lds = 0;
  if (t.lds_bytes >= 0) {
    lds = (unsigned)t.lds_bytes;
  } else if (big || (n_in == 2 && n_out == 2 && total_bytes >= (64l << 20))) {
    // (a ring reduce step, 2 -> 2, gains from its cap of 5 already at 16 MiB per buffer: 7 steps
    // over distinct 32 MiB chunks 150 -> 146 us, the same buffers again and again at 16 MiB per
    // buffer 6.5 -> 6.9 TB/s; 2 -> 1, 3 -> 1, 4 -> 1 and 8 -> 1 of that size lose 1-4 % under theirs)
    const int streams = n_in + n_out;
    int wgs = (20 + streams / 2) / streams;
    wgs = std::max(2, std::min(8, wgs));
    // the 8-bit floats spend 16 conversions per input pack: they need more wavefronts to hide
    // that arithmetic behind the loads (8 -> 1 at 256 MiB: 6.2 TB/s with 2 workgroups, 6.35 with 4)
    if (es == 1 && n_in > 1) wgs = std::max(wgs, 4);
    if (wgs < 8) lds = std::min(65536u, (unsigned)(160 * 1024 / wgs) - 256u);
  }
  // Workgroup -> chunk rotation (rotated_chunk in reduce_copy_kernel.h) wherever the launch has one
  // workgroup per 4 KiB chunk and the operands are treated as streams (48 MiB in all and more).  It pays
  // when the data comes from HBM and costs when it sits in the Infinity Cache.  bf16 on operands in
  // separate allocations, TB/s without / with: the same buffers again and again, 128 MiB per buffer:
  // 8 -> 1 6.69 / 6.95, 2 -> 2 6.81 / 7.20, 1 -> 1 6.61 / 6.91; 32 MiB per buffer (cache-resident):
  // 2 -> 2 6.06 / 6.00, 1 -> 1 5.85 / 5.50, 4 -> 1 6.27 / 5.66; walks over distinct buffers (what a collective
  // step sees), 32 MiB: 2 -> 2 5.67 / 6.02, 1 -> 1 5.73 / 5.92, 2 -> 1 5.97 / 6.23; 16 MiB: 5.44 / 5.76, 5.19 / 5.27,
  // 5.21 / 5.47.
  // Not for operands of 4 GiB and more each: there the outcome turns on address bits beyond those the
  // rotation was fitted to.  Slices of one 160 GiB allocation, operand size / distance between operands,
  // TB/s without / with: copy 8 GiB / 8 GiB 6.68 / 6.75 but 8 / 32 6.66 / 6.14 and 16 / 16 6.67 / 5.68;
  // 2 -> 1 4 / 4 6.28 / 6.69 but 4 / 32 6.64 / 6.08, 8 / 32 6.64 / 5.74, 16 / 16 6.53 / 5.96; 4 -> 1 4 / 4 5.93 / 6.51 but
  // 4 / 32 6.09 / 5.67, 16 / 32 6.12 / 5.57.  Without it every such case stays within 5.9-6.7; at 1 GiB per
  // operand the rotation wins or ties at every distance (4 -> 1: 6.03 / 6.27 .. 6.10 / 6.25).
  p.rotate = total_bytes >= (48l << 20) && count * es < (4l << 30) && unroll <= 1 && grid == chunks && t.rotate != 0;
  if (t.rotate > 0 && unroll <= 1 && grid == chunks) p.rotate = 1;
  hipStream_t s = (hipStream_t)stream;
  if (n_in == 1) return launch_copy(es, unroll, aligned, mem, (unsigned)grid, lds, s, p);
  switch (dtype) {
    case PCCL_F32: return launch_typed<PCCL_F32>(compute, n_in, unroll, aligned, mem, (unsigned)grid, lds, s, p);
    case PCCL_I32: return launch_typed<PCCL_I32>(compute, n_in, unroll, aligned, mem, (unsigned)grid, lds, s, p);
    case PCCL_BF16: return launch_typed<PCCL_BF16>(compute, n_in, unroll, aligned, mem, (unsigned)grid, lds, s, p);
    case PCCL_F16: return launch_typed<PCCL_F16>(compute, n_in, unroll, aligned, mem, (unsigned)grid, lds, s, p);
    case PCCL_F8E4M3: return launch_typed<PCCL_F8E4M3>(compute, n_in, unroll, aligned, mem, (unsigned)grid, lds, s, p);
    case PCCL_F8E5M2: return launch_typed<PCCL_F8E5M2>(compute, n_in, unroll, aligned, mem, (unsigned)grid, lds, s, p);
    case PCCL_F64: return launch_typed<PCCL_F64>(compute, n_in, unroll, aligned, mem, (unsigned)grid, lds, s, p);
    default: return launch_typed<PCCL_U32>(compute, n_in, unroll, aligned, mem, (unsigned)grid, lds, s, p);
  }
}
