// HBM-to-HBM byte copy shared by put/get/broadcast/alltoall at workgroup,
// wavefront and single-lane granularity.
//
// The reference moves 8 bytes per lane per step through uncached stores
// (memcpy_wg / memcpy_wave / memcpy, library/src/util.hpp:248-325).  Here a
// group of `nthr` lanes moves 16 bytes per lane per access, four accesses in
// flight per lane: destination-aligned global_store_dwordx4, sources read as
// dwordx4 at whatever 4-byte alignment they have, and byte-misaligned
// sources re-aligned in registers with v_alignbyte_b32.  Semantics are exactly
// memcpy(dst, src, n) for non-overlapping ranges.
#ifndef ROCSHMEM_MI355X_DEVICE_COPY_HPP
#define ROCSHMEM_MI355X_DEVICE_COPY_HPP

#include "state.hpp"
#include "sync.hpp"
#include "wave.hpp"

namespace rocshmem {
namespace detail {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));

constexpr int kCopyUnroll = 4;
// Copies at least this large bypass cache allocation (nt loads and stores):
// the payload is touched once and is larger than what the L2 would keep.
constexpr size_t kNonTemporalBytes = 256 * 1024;

template <bool kNt>
__device__ __forceinline__ u32x4 load_vec(const u32x4 *p) {
  if constexpr (kNt) return __builtin_nontemporal_load(p);
  return *p;
}
template <bool kNt>
__device__ __forceinline__ void store_vec(u32x4 v, u32x4 *p) {
  if constexpr (kNt) {
    __builtin_nontemporal_store(v, p);
  } else {
    *p = v;
  }
}

// dst and src both 16-byte aligned; kDepth loads are in flight per lane.
template <bool kNt, int kDepth = kCopyUnroll>
__device__ __forceinline__ void copy_vec_aligned(u32x4 *__restrict__ d,
                                                 const u32x4 *__restrict__ s, size_t nvec,
                                                 uint32_t tid, uint32_t nthr) {
  size_t i = tid;
  const size_t step = nthr;
  for (; i + (kDepth - 1) * step < nvec; i += kDepth * step) {
    u32x4 v[kDepth];
#pragma unroll
    for (int k = 0; k < kDepth; ++k) v[k] = load_vec<kNt>(&s[i + k * step]);
#pragma unroll
    for (int k = 0; k < kDepth; ++k) store_vec<kNt>(v[k], &d[i + k * step]);
  }
  for (; i < nvec; i += step) store_vec<kNt>(load_vec<kNt>(&s[i]), &d[i]);
}

// dst 16-byte aligned, src 4-byte aligned.
__device__ __forceinline__ void copy_vec_src_dword(u32x4 *__restrict__ d,
                                                   const char *__restrict__ s, size_t nvec,
                                                   uint32_t tid, uint32_t nthr) {
  const u32x4_a4 *sv = reinterpret_cast<const u32x4_a4 *>(s);
  size_t i = tid;
  const size_t step = nthr;
  for (; i + (kCopyUnroll - 1) * step < nvec; i += kCopyUnroll * step) {
    u32x4 v[kCopyUnroll];
#pragma unroll
    for (int k = 0; k < kCopyUnroll; ++k) v[k] = sv[i + k * step];
#pragma unroll
    for (int k = 0; k < kCopyUnroll; ++k) d[i + k * step] = v[k];
  }
  for (; i < nvec; i += step) d[i] = sv[i];
}

// dst 16-byte aligned, src at byte offset `shift` (1..3) past a 4-byte
// boundary.  Each lane reads the five aligned dwords that cover its 16
// destination bytes and funnels them together.  The caller guarantees that
// the dword holding the last source byte of every vector lies inside the
// source range's enclosing aligned dwords (true for any in-bounds source:
// the fifth dword always contains at least one requested byte).
__device__ __forceinline__ void copy_vec_src_bytes(u32x4 *__restrict__ d,
                                                   const char *__restrict__ s, size_t nvec,
                                                   uint32_t tid, uint32_t nthr) {
  const uint32_t shift = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(s) & 3u);
  const uint32_t *sw = reinterpret_cast<const uint32_t *>(s - shift);
  for (size_t i = tid; i < nvec; i += nthr) {
    const u32x4_a4 *lo = reinterpret_cast<const u32x4_a4 *>(sw + 4 * i);
    u32x4 w = *lo;
    uint32_t w4 = sw[4 * i + 4];
    u32x4 o;
    o.x = __builtin_amdgcn_alignbyte(w.y, w.x, shift);
    o.y = __builtin_amdgcn_alignbyte(w.z, w.y, shift);
    o.z = __builtin_amdgcn_alignbyte(w.w, w.z, shift);
    o.w = __builtin_amdgcn_alignbyte(w4, w.w, shift);
    d[i] = o;
  }
}

// dst 16-byte aligned, src at any byte offset, group-uniform arguments: the
// hardware reads a 16-byte vector at any byte address (unaligned access is
// enabled for global memory), so the pass structure of stream_copy_uniform
// carries over with per-lane global loads in place of buffer loads.
typedef u32x4 u32x4_a1 __attribute__((aligned(1)));
template <bool kNt, int U>
__device__ __forceinline__ void stream_copy_src_unaligned(char *d, const char *s, size_t nbytes,
                                                          uint32_t tid, uint32_t nthr,
                                                          size_t first_pass = 0,
                                                          size_t pass_step = 1) {
  const size_t access_bytes = static_cast<size_t>(nthr) * 16u;
  const size_t pass_bytes = access_bytes * U;
  const size_t mine = static_cast<size_t>(tid) * 16u;
  // This group takes passes first_pass, first_pass + pass_step, ...; the last
  // pass of the range may be partial.
  for (size_t b = first_pass * pass_bytes; b < nbytes; b += pass_step * pass_bytes) {
    if (b + pass_bytes <= nbytes) {
      u32x4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const u32x4_a1 *p = reinterpret_cast<const u32x4_a1 *>(s + b + u * access_bytes + mine);
        if constexpr (kNt) {
          v[u] = __builtin_nontemporal_load(p);
        } else {
          v[u] = *p;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        store_vec<kNt>(v[u], reinterpret_cast<u32x4 *>(d + b + u * access_bytes + mine));
    } else {
      for (size_t at = b + mine; at < nbytes; at += access_bytes)
        *reinterpret_cast<u32x4 *>(d + at) = *reinterpret_cast<const u32x4_a1 *>(s + at);
    }
  }
}

// memcpy(dst, src, n) executed cooperatively by lanes tid = 0..nthr-1, for
// per-lane (possibly different in every lane) arguments: the thread-level
// put/get path.  No barrier inside.
__device__ __forceinline__ void group_copy(void *dst, const void *src, size_t n, uint32_t tid,
                                           uint32_t nthr) {
  char *d = static_cast<char *>(dst);
  const char *s = static_cast<const char *>(src);
  if (n < 64) {
    for (size_t i = tid; i < n; i += nthr) d[i] = s[i];
    return;
  }
  // Head: bring the destination to a 16-byte boundary.
  size_t head = (16u - (reinterpret_cast<uintptr_t>(d) & 15u)) & 15u;
  for (size_t i = tid; i < head; i += nthr) d[i] = s[i];
  d += head;
  s += head;
  n -= head;

  size_t nvec = n / 16;
  size_t body = nvec * 16;
  uintptr_t smis = reinterpret_cast<uintptr_t>(s) & 15u;
  u32x4 *dv = reinterpret_cast<u32x4 *>(d);
  if (smis == 0) {
    if (body >= kNonTemporalBytes) {
      copy_vec_aligned<true>(dv, reinterpret_cast<const u32x4 *>(s), nvec, tid, nthr);
    } else {
      copy_vec_aligned<false>(dv, reinterpret_cast<const u32x4 *>(s), nvec, tid, nthr);
    }
  } else if ((smis & 3u) == 0) {
    copy_vec_src_dword(dv, s, nvec, tid, nthr);
  } else {
    copy_vec_src_bytes(dv, s, nvec, tid, nthr);
  }
  // Tail: fewer than 16 bytes.
  size_t tail = n - body;
  for (size_t i = tid; i < tail; i += nthr) d[body + i] = s[body + i];
}

constexpr int kStreamUnroll = 8;          // 16-byte accesses per lane per pass
constexpr int kRawBufferFlags = 0x00020000;  // untyped 32-bit data, no swizzle
// Cache-policy bit of a raw-buffer access: sc1.  A store that carries it is
// written through this XCD's L2 to memory (visible to the other XCDs once the
// storing wave's s_waitcnt vmcnt(0) has passed); streaming stores run as fast
// with it as without (write-only probe: plain, sc0, sc1, nt within 2 %).
constexpr int kWriteThrough = 16;

// Descriptor over [base, base + bytes) for a group whose lanes all pass the
// same `base` and `bytes`.  Both go through readfirstlane here even though the
// callers' values are uniform already: when the compiler has moved such a
// value into vector registers (a 64-bit unsigned compare has no scalar form,
// and everything computed from its result follows it to the vector unit) it
// no longer knows the descriptor is uniform and wraps every buffer access in
// a loop over the distinct values it might hold - a dozen extra instructions
// per access, which cost the 1 -> 15 broadcast a sixth of its bandwidth.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t uniform_rsrc(const void *base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(uniform(base)), 0, uniform(bytes),
                                           kRawBufferFlags);
}

// Lockstep pacing of a large stream shared by all workgroups of a grid.
//
// Left to themselves, the workgroups of a streaming kernel drift apart, and at
// any moment some memory channels are asked for more than they can deliver
// while others idle: a plain copy of 8 x 256 MiB runs at 5.9-6.0 TB/s on
// MI355X although reads alone reach 6.8-7.1 and writes alone 6.3-6.6.  Time is
// therefore cut into slots of `period` ticks of the 100 MHz constant clock,
// which every workgroup can read: a workgroup issues the loads of a pass in
// one slot and its stores in the next.  All workgroups then start each burst
// at the same instant, and the bursts sweep one compact window of every array.
// Which slot is whose differs by the kind of stream: see make_pacer (copies:
// neighbouring XCDs a slot apart, half the chip reading while the other half
// writes) and make_anchored_pacer (reductions: the whole chip in phase).
//
// The slots are a schedule, not a gate: a wave keeps the start time of its
// next burst, waits for it when it is early and goes at once when it is late.
// With a rate the memory system can sustain everybody is on time and the
// stream runs at that rate; with a rate beyond it everybody runs late, nobody
// waits, and the stream keeps most of the gain of its aligned start (8 -> 8
// fp32 reduction, bare kernel, one card: 6.00 TB/s free, 6.21 paced at 6.2,
// 6.33 at 6.7, 6.22 at 7.0, 6.10 at 9.0 TB/s).  Gating on the slot's parity
// instead (wait whenever the clock is in the other kind of slot) reaches the
// same peak, but a wave that misses its slot then waits a whole slot for the
// next, and 2 % beyond the best rate the stream falls to 4.9-5.4 TB/s.
//
// The schedule assumes that every workgroup of the grid is resident: those of
// a grid larger than the chip would wait for slots sized for all of them while
// only some run (half the rate for twice the chip).  make_pacer's callers
// check that.  period == 0: no pacing.  Every wait ends by itself: the clock
// advances.
struct Pacer {
  uint32_t period;   // ticks per slot; 0 = not paced
  uint64_t next;     // clock value at which the next burst of this wave is due
  // Waits for the burst that is due, then books the next one `step` ticks later.
  __device__ __forceinline__ void wait(uint32_t step) {
    if (period == 0) return;
    // (-DROCSHMEM_AB_NO_SLEEP: an A/B build for measurements that polls the clock without sleeping)
#ifdef ROCSHMEM_AB_NO_SLEEP
    while (static_cast<int64_t>(wall_clock64() - next) < 0) {}
#else
    while (static_cast<int64_t>(wall_clock64() - next) < 0) __builtin_amdgcn_s_sleep(2);
#endif
    next += step;
  }
  __device__ __forceinline__ void wait_slot() { wait(period); }
};

// `slot_bytes`: what all workgroups of the grid move in one slot (loads of one
// half plus stores of the other).  Too few or too many ticks per slot: no
// pacing.  The first burst (loads) is due at the start of the first slot of
// this XCD's load parity that has not ended yet.
__device__ __forceinline__ Pacer make_pacer(uint32_t bytes_per_tick, uint64_t slot_bytes) {
  Pacer p{0u, 0u};
  if (bytes_per_tick == 0) return p;
  const uint64_t period = (slot_bytes + bytes_per_tick - 1) / bytes_per_tick;
  if (period < 64 || period > 50000) return p;
  p.period = static_cast<uint32_t>(period);
  // XCC_ID: the XCD this workgroup runs on
  const uint32_t parity = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 1u;
  uint64_t slot = wall_clock64() / period;
  slot += (static_cast<uint32_t>(slot) ^ parity) & 1u;
  p.next = slot * period;
  return p;
}

// The slots of a reduction (reduce_vectors).  The whole chip is in phase here: every
// workgroup issues the loads of a pass in one slot and its stores in the next, so that memory
// serves reads alone for a slot and writes alone for the next.  The slot grid is anchored at
// the launch (the clock rounded up to kPaceGranuleTicks, which workgroups that start within
// 2 us of each other agree on) and a reduction of P passes per workgroup takes 2 P slots.
// 8 -> 8 fp32 reduction of 2^26 elements, 32 workgroups of 1024 lanes per PE, one card, best
// rate of each: 6030-6080 GB/s running free; 6160-6170 with neighbouring XCDs a slot apart
// (one half of the chip loading while the other stores, which takes a seventeenth slot in
// which half the chip works alone; -DROCSHMEM_AB_ALTERNATE_PHASE builds that for
// measurements), 6423-6445 with the odd XCDs' first pass split in two halves that fill that
// slot at either end; 6550-6576 in phase.  A mixed stream costs every request more at the
// memory side (a read 2500-3100 L2 cycles against 1660-2250 in a stream of reads alone) than
// the burst of one kind that the whole chip issues at once.  A reduction's pass is eight
// rounds of loads, each waiting for the one before (the fold), and one burst of stores; a
// copy's pass is one round of each, and copies run best free (make_pacer, off by default).
constexpr uint32_t kPaceGranuleTicks = 200;   // (100, 400 and 800 ticks measured the same within 0.5 %)
__device__ __forceinline__ Pacer make_anchored_pacer(uint32_t bytes_per_tick, uint64_t slot_bytes) {
  Pacer p{0u, 0u};
  if (bytes_per_tick == 0) return p;
  const uint64_t period = (slot_bytes + bytes_per_tick - 1) / bytes_per_tick;
  if (period < 64 || period > 50000) return p;
  p.period = static_cast<uint32_t>(period);
  p.next = (wall_clock64() + kPaceGranuleTicks - 1) / kPaceGranuleTicks * kPaceGranuleTicks;
#ifdef ROCSHMEM_AB_ALTERNATE_PHASE
  if (__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 1u) p.next += period;   // XCC_ID
#endif
  return p;
}

__device__ __forceinline__ uint64_t grid_workgroups() {
  return static_cast<uint64_t>(gridDim.x) * gridDim.y * gridDim.z;
}

// This grid fills the chip and all of its workgroups run at the same time (what a
// paced stream needs).
__device__ __forceinline__ bool grid_is_resident() {
  const uint64_t wgs = grid_workgroups();
  // A compute unit holds 1024 lanes of these kernels (16 waves at 65-128 vector registers) in
  // whole workgroups: one of 640 lanes, not one and a half (384 workgroups of 640 lanes passed
  // a test on lanes alone, a third of them waited for a free compute unit, and the paced
  // reduction ran at 3.1 TB/s against 4.9 running free).
  const uint32_t per_cu = 1024u / flat_block_size();
  const uint64_t cus = g_state.pace_max_grid_lanes / 1024u;
  return wgs >= g_state.pace_min_grid_workgroups && wgs <= cus * per_cu;
}

// Body of a group copy whose arguments are the same in every lane
// (workgroup- and wave-collective calls): `d` 16-byte aligned, `s` 4-byte
// aligned, `nbytes` a multiple of 16.  One pass moves U*nthr*16
// consecutive bytes (128 KiB for 1024 lanes and U = 8): all loads of the pass are
// issued before its stores.  Addresses are "descriptor + scalar offset +
// tid*16", so no lane carries a 64-bit address, and the descriptor's size
// field turns the last partial pass into the same code (accesses beyond
// `valid` load zeros and store nothing).
// (`pacer` by reference: a caller that moves several ranges one after the other keeps one
// schedule across them.)
template <int kAux, int U, int kStoreAux = kAux>
__device__ __forceinline__ void stream_copy_paced(char *d, const char *s, size_t nbytes,
                                                  uint32_t tid, uint32_t nthr, size_t first_pass,
                                                  size_t pass_step, Pacer &pacer) {
  const uint32_t lane_off = tid * 16u;
  const uint32_t access_bytes = nthr * 16u;
  const uint32_t pass_bytes = access_bytes * U;
  // This group takes passes first_pass, first_pass + pass_step, ...
  const size_t step_bytes = pass_step * pass_bytes;
  for (size_t b = first_pass * pass_bytes; b < nbytes; b += step_bytes) {
    const size_t left = nbytes - b;
    const int valid = static_cast<int>(left < pass_bytes ? left : pass_bytes);
    __amdgpu_buffer_rsrc_t rs = uniform_rsrc(s + b, valid);
    __amdgpu_buffer_rsrc_t rd = uniform_rsrc(d + b, valid);
    u32x4 v[U];
    pacer.wait_slot();
#pragma unroll
    for (int u = 0; u < U; ++u)
      v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane_off, u * access_bytes, kAux);
    if (pacer.period) {
      // the data first, then the slot: stores leave together at the slot's start
      __builtin_amdgcn_s_waitcnt(0);
      pacer.wait_slot();
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      __builtin_amdgcn_raw_buffer_store_b128(v[u], rd, lane_off, u * access_bytes, kStoreAux);
  }
}

// Stores of messages from 64 KiB on are written through even when the message is too short for
// the streaming policy: the bytes have to reach memory before another XCD can see them, and what
// has been written through the next quiet does not have to write back (8 PEs, workgroup puts of
// 64 / 128 KiB: 5815 / 5800 GB/s with stores that stay in the L2 until then, 5958 / 5974 written
// through).  Shorter messages keep plain stores: written through, a put of 4 KiB gained 1 % in a
// stream of them, but a call on its own ended later (broadcast, alltoall and fcollect of 4-32 KiB
// among 8 PEs: 5.8-6.2 -> 6.0-6.6 us).
constexpr size_t kWriteThroughFromBytes = 64 * 1024;
template <int kAux, int U, int kStoreAux = kAux>
__device__ __forceinline__ void stream_copy_uniform(char *d, const char *s, size_t nbytes,
                                                    uint32_t tid, uint32_t nthr,
                                                    size_t first_pass = 0, size_t pass_step = 1,
                                                    Pacer pacer = Pacer{0u, 0u}) {
  stream_copy_paced<kAux, U, kStoreAux>(d, s, nbytes, tid, nthr, first_pass, pass_step, pacer);
}

// Picks the pass depth by message size, so that a message that one or two
// accesses of the group cover does not issue eight (six or seven of them
// entirely out of range).
__device__ __forceinline__ void stream_copy_sized(char *d, const char *s, size_t nbytes,
                                                  uint32_t tid, uint32_t nthr, bool part_of_a_stream = false) {
  const size_t access_bytes = static_cast<size_t>(nthr) * 16u;
  if (nbytes >= kNonTemporalBytes) {
    stream_copy_uniform<2 /* nt */, kStreamUnroll>(d, s, nbytes, tid, nthr);
  } else if (part_of_a_stream) {
    // a short share of a transfer that is large as a whole: touched once, like the whole
    if (nbytes <= access_bytes) {
      stream_copy_uniform<2, 1>(d, s, nbytes, tid, nthr);
    } else if (nbytes <= 2 * access_bytes) {
      stream_copy_uniform<2, 2>(d, s, nbytes, tid, nthr);
    } else if (nbytes <= 4 * access_bytes) {
      stream_copy_uniform<2, 4>(d, s, nbytes, tid, nthr);
    } else {
      stream_copy_uniform<2, kStreamUnroll>(d, s, nbytes, tid, nthr);
    }
  } else if (nbytes <= access_bytes) {
    stream_copy_uniform<0, 1>(d, s, nbytes, tid, nthr);
  } else if (nbytes <= 2 * access_bytes) {
    stream_copy_uniform<0, 2>(d, s, nbytes, tid, nthr);
  } else if (nbytes <= 4 * access_bytes) {
    if (nbytes >= kWriteThroughFromBytes) {
      stream_copy_uniform<0, 4, kWriteThrough>(d, s, nbytes, tid, nthr);
    } else {
      stream_copy_uniform<0, 4>(d, s, nbytes, tid, nthr);
    }
  } else if (nbytes >= kWriteThroughFromBytes) {
    stream_copy_uniform<0, kStreamUnroll, kWriteThrough>(d, s, nbytes, tid, nthr);
  } else {
    stream_copy_uniform<0, kStreamUnroll>(d, s, nbytes, tid, nthr);
  }
}

// Bytes in front of the vector body of a copy of `n` bytes to `d`: up to the
// next 16-byte boundary, for a message of some size up to the next 128-byte
// boundary (every wave store then covers whole cache lines) and for a large
// one up to the next 1 KiB boundary (the 1 KiB that the 64 lanes of a wave
// store with one instruction then never straddles two).  Measured on MI355X,
// 8 x 192 MiB put as 64 MiB messages: 4.98 TB/s with the body starting 16
// bytes past a 128-byte boundary, 5.94 at a 128-byte boundary that is not a
// 1 KiB boundary, 6.1 at a 1 KiB boundary; a 1 -> 7 broadcast of 64 MiB takes
// 146 us from a 128-byte and 138 us from a 1 KiB boundary.
constexpr size_t kStoreChunkBytes = 1024;
__device__ __forceinline__ size_t stream_head(const char *d, size_t n) {
  const uintptr_t at = reinterpret_cast<uintptr_t>(d);
  const uintptr_t boundary = n >= 65536 ? kStoreChunkBytes : n >= 4096 ? 128u : 16u;
  return (boundary - (at & (boundary - 1))) & (boundary - 1);
}

// memcpy(dst, src, n) by lanes tid = 0..nthr-1 of a group that passes the
// same (dst, src, n) in every lane.
__device__ __forceinline__ void group_copy_uniform(void *dst, const void *src, size_t n,
                                                   uint32_t tid, uint32_t nthr,
                                                   bool part_of_a_stream = false) {
  char *d = static_cast<char *>(dst);
  const char *s = static_cast<const char *>(src);
  if (n < 64) {
    for (size_t i = tid; i < n; i += nthr) d[i] = s[i];
    return;
  }
  const size_t head = stream_head(d, n);
  for (size_t i = tid; i < head; i += nthr) d[i] = s[i];
  d += head;
  s += head;
  n -= head;
  const size_t body = n & ~static_cast<size_t>(15);
  if ((reinterpret_cast<uintptr_t>(s) & 3u) == 0) {
    stream_copy_sized(d, s, body, tid, nthr, part_of_a_stream);
  } else {
    if (body >= kNonTemporalBytes) {
      stream_copy_src_unaligned<true, kStreamUnroll>(d, s, body, tid, nthr);
    } else {
      stream_copy_src_unaligned<false, kCopyUnroll>(d, s, body, tid, nthr);
    }
  }
  for (size_t i = body + tid; i < n; i += nthr) d[i] = s[i];
}

// memcpy(dst, src, n) shared by `parts` groups that all pass the same
// arguments and their own `part`: a large copy between mutually aligned
// buffers is dealt pass by pass (the groups running at one moment then sweep
// one compact window of both buffers), anything else is cut into contiguous
// ranges.  Complete when every part has returned.
__device__ __forceinline__ void group_copy_dealt(void *dst, const void *src, size_t n,
                                                 uint32_t tid, uint32_t nthr, size_t part,
                                                 size_t parts, uint32_t pace_bytes_per_tick = 0) {
  if (parts <= 1) {
    group_copy_uniform(dst, src, n, tid, nthr);
    return;
  }
  char *d = static_cast<char *>(dst);
  const char *s = static_cast<const char *>(src);
  const size_t pass_bytes = static_cast<size_t>(nthr) * 16u * kStreamUnroll;
  // The vector path stores 16-byte aligned and loads at any 4-byte alignment.
  const bool coaligned =
      ((reinterpret_cast<uintptr_t>(d) ^ reinterpret_cast<uintptr_t>(s)) & 3u) == 0;
  if (n >= 2 * parts * pass_bytes) {
    const size_t head = stream_head(d, n);
    const size_t body = (n - head) & ~static_cast<size_t>(15);
    if (part == 0) {
      for (size_t i = tid; i < head; i += nthr) d[i] = s[i];
      for (size_t i = head + body + tid; i < n; i += nthr) d[i] = s[i];
    }
    if (coaligned) {
      // Paced when the library holds a rate for copies, the grid fills the chip and every
      // workgroup has passes enough for the start of the slots to disappear: a call's first
      // burst waits for the next slot of its kind, up to two slots, and the schedule brings 2 %
      // (8 PEs, 32 x 1024 lanes per PE, at 67000: one message of 256 MiB per PE, 64 passes per
      // workgroup, 6413-6437 GB/s free and 6519-6569 paced; four of 64 MiB, 16 passes each,
      // 6396-6431 free and 6104-6212 paced).
      Pacer pacer{0u, 0u};
      if (pace_bytes_per_tick != 0 && body >= 64 * parts * pass_bytes && grid_is_resident())
        pacer = make_pacer(pace_bytes_per_tick, grid_workgroups() * pass_bytes);
      stream_copy_uniform<2 /* nt */, kStreamUnroll>(d + head, s + head, body, tid, nthr, part, parts,
                                                     pacer);
    } else {
      stream_copy_src_unaligned<true, kStreamUnroll>(d + head, s + head, body, tid, nthr, part, parts);
    }
  } else {
    // (a division of 32-bit values when they are: a workgroup that lives for one share of a
    // few KiB should not spend its time in a 64-bit division routine)
    size_t share = (n >> 32) == 0 && (parts >> 32) == 0
                       ? (static_cast<uint32_t>(n) + static_cast<uint32_t>(parts) - 1) / static_cast<uint32_t>(parts)
                       : (n + parts - 1) / parts;
    share = (share + 255) / 256 * 256;
    size_t b = share * part, e = b + share;
    if (b > n) b = n;
    if (e > n) e = n;
    if (e > b) group_copy_uniform(d + b, s + b, e - b, tid, nthr, n >= kNonTemporalBytes);
  }
}

__device__ __forceinline__ void wg_copy(void *dst, const void *src, size_t n) {
  // Workgroup-collective: the arguments are the same in every lane.
  group_copy_uniform(uniform(dst), uniform(src), uniform(n), flat_thread_id(), flat_block_size());
}

// One copy shared by `nshards` workgroups (workgroup-collective in each).
__device__ __forceinline__ void wg_copy_shard(void *dst, const void *src, size_t n, int shard,
                                              int nshards, uint32_t pace_bytes_per_tick = 0) {
  shard = uniform(shard);
  nshards = uniform(nshards);
  if (nshards <= 0 || shard < 0 || shard >= nshards) return;
  group_copy_dealt(uniform(dst), uniform(src), uniform(n), flat_thread_id(), flat_block_size(),
                   static_cast<size_t>(shard), static_cast<size_t>(nshards),
                   uniform(pace_bytes_per_tick));
}

__device__ __forceinline__ void wave_copy(void *dst, const void *src, size_t n) {
  // All lanes of the calling wave take part (wave-collective call).
  group_copy_uniform(uniform(dst), uniform(src), uniform(n), lane_id(), kWaveSize);
}

// One naturally aligned element moved with device-coherent accesses (agent-scope
// relaxed atomics: the store is written through this XCD's L2, the load does
// not trust a line another XCD may have changed).  Single-element puts and
// gets are what programs signal and poll with - p on one PE, wait_until or a
// g loop on another, no quiet in between (reference: ping_pong_tester.cpp:
// 48-57) - so they must not sit in a write-back cache or be served from a
// stale line until the kernel ends.
template <typename W>
__device__ __forceinline__ void coherent_store(void *dst, W bits) {
  __hip_atomic_store(static_cast<W *>(dst), bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename W>
__device__ __forceinline__ W coherent_load(const void *src) {
  return __hip_atomic_load(static_cast<const W *>(src), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One naturally aligned piece of W bytes, if `take`: load now, store later.
template <typename W>
struct LanePiece {
  W bits;
  bool take;
  __device__ __forceinline__ void load(const char *s, bool t) {
    take = t;
    if (take) bits = *reinterpret_cast<const W *>(s);
  }
  __device__ __forceinline__ void store(char *d) const {
    if (take) *reinterpret_cast<W *>(d) = bits;
  }
};

// memcpy(d, s, n) by one lane for buffers that are aligned alike modulo 16
// (n >= 32).  A lane has no neighbours to share the message with, so what
// counts is how many memory round trips it makes: the bytes in front of the
// first and behind the last 16-byte vector are moved as at most four
// naturally aligned pieces each, all loaded before any is stored, and the
// vectors go eight at a time, the last partial group included.  A 1000-byte
// message takes 9 round trips this way, 21 when every leftover vector and
// byte makes its own.
__device__ __forceinline__ void lane_copy_coaligned(char *d, const char *s, size_t n) {
  constexpr int kDepth = 2 * kCopyUnroll;
  const uint32_t lead = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(d)) & 15u;
  const size_t head = (16u - lead) & 15u;
  const size_t nvec = (n - head) / 16;
  const size_t tail = n - head - nvec * 16;
  {
    // Head pieces rise in size (1, 2, 4, 8 bytes bring the address to the next
    // boundary), tail pieces fall (8, 4, 2, 1 bytes of what is left).
    LanePiece<uint8_t> h1, t1;
    LanePiece<uint16_t> h2, t2;
    LanePiece<uint32_t> h4, t4;
    LanePiece<uint64_t> h8, t8;
    size_t o = 0;
    h1.load(s + o, (head & 1u) != 0);
    const size_t o1 = o;
    o += head & 1u;
    h2.load(s + o, (head & 2u) != 0);
    const size_t o2 = o;
    o += head & 2u;
    h4.load(s + o, (head & 4u) != 0);
    const size_t o4 = o;
    o += head & 4u;
    h8.load(s + o, (head & 8u) != 0);
    const size_t o8 = o;
    size_t q = head + nvec * 16;
    t8.load(s + q, (tail & 8u) != 0);
    const size_t q8 = q;
    q += tail & 8u;
    t4.load(s + q, (tail & 4u) != 0);
    const size_t q4 = q;
    q += tail & 4u;
    t2.load(s + q, (tail & 2u) != 0);
    const size_t q2 = q;
    q += tail & 2u;
    t1.load(s + q, (tail & 1u) != 0);
    const size_t q1 = q;
    h1.store(d + o1);
    h2.store(d + o2);
    h4.store(d + o4);
    h8.store(d + o8);
    t8.store(d + q8);
    t4.store(d + q4);
    t2.store(d + q2);
    t1.store(d + q1);
  }
  const u32x4 *sv = reinterpret_cast<const u32x4 *>(s + head);
  u32x4 *dv = reinterpret_cast<u32x4 *>(d + head);
  size_t i = 0;
  for (; i + kDepth <= nvec; i += kDepth) {
    u32x4 v[kDepth];
#pragma unroll
    for (int k = 0; k < kDepth; ++k) v[k] = sv[i + k];
#pragma unroll
    for (int k = 0; k < kDepth; ++k) dv[i + k] = v[k];
  }
  const size_t left = nvec - i;
  if (left) {
    u32x4 v[kDepth - 1];
#pragma unroll
    for (int k = 0; k < kDepth - 1; ++k)
      if (static_cast<size_t>(k) < left) v[k] = sv[i + k];
#pragma unroll
    for (int k = 0; k < kDepth - 1; ++k)
      if (static_cast<size_t>(k) < left) dv[i + k] = v[k];
  }
}

// Single-lane copy used by the thread-level put/get: the common 4- and 8-byte
// naturally aligned messages are one coherent load and one coherent store.
__device__ __forceinline__ void lane_copy(void *dst, const void *src, size_t n) {
  uintptr_t both = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src);
  if (n == 8 && (both & 7u) == 0) {
    coherent_store<uint64_t>(dst, coherent_load<uint64_t>(src));
  } else if (n == 4 && (both & 3u) == 0) {
    coherent_store<uint32_t>(dst, coherent_load<uint32_t>(src));
  } else if (n >= 32 && n < kNonTemporalBytes &&
             ((reinterpret_cast<uintptr_t>(dst) ^ reinterpret_cast<uintptr_t>(src)) & 15u) == 0) {
    lane_copy_coaligned(static_cast<char *>(dst), static_cast<const char *>(src), n);
  } else {
    group_copy(dst, src, n, 0u, 1u);
  }
}

}  // namespace detail
}  // namespace rocshmem

#endif
