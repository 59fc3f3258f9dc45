/**
 * Device-side support library for the kernels the HIP lowering emits (gfx950 / CDNA4, wavefront 64).
 *
 * Everything here is written for one target only. The lowering emits one `extern "C" __global__` function
 * per op description; that function is a thin, fully unrolled composition of the pieces below:
 *   - dtype traits: how each element type of the op description is stored in memory, which register type
 *     it is computed in, and how a result is rounded back to the declared type after every op (the CPU
 *     pipeline of the reference computes each op in its declared result type),
 *   - 128-bit vector global loads/stores,
 *   - the per-op scalar semantics (tosa/linalg/libm lowering of the reference CPU pipeline),
 *   - row-group reductions: xor butterfly inside a wavefront (DPP for the quad steps), LDS across wavefronts.
 *
 * Compiled by hiprtc, so it includes nothing.
 */
#pragma once

namespace akg {

typedef unsigned char u8;
typedef signed char s8;
typedef unsigned short u16;
typedef unsigned int u32;
typedef unsigned long long u64;
typedef _Float16 half_t;
typedef __bf16 bfloat_t;

constexpr int kWaveSize = 64;

#define AKG_DEV __device__ __forceinline__

// ---------------------------------------------------------------------------------------------------------
// dtype traits. `storage` is the in-memory element, `compute` the register type, `rnd` rounds a compute
// value to the nearest representable value of the declared type (round-to-nearest-even, what arith.truncf
// does in the reference CPU pipeline).
// ---------------------------------------------------------------------------------------------------------
struct f32 {
  typedef float storage;
  typedef float compute;
  static AKG_DEV compute rnd(compute x) { return x; }
  static AKG_DEV compute load(storage s) { return s; }
  static AKG_DEV storage store(compute x) { return x; }
};
struct f64 {
  typedef double storage;
  typedef double compute;
  static AKG_DEV compute rnd(compute x) { return x; }
  static AKG_DEV compute load(storage s) { return s; }
  static AKG_DEV storage store(compute x) { return x; }
};
struct f16 {
  typedef half_t storage;
  typedef float compute;
  static AKG_DEV compute rnd(compute x) { return static_cast<float>(static_cast<half_t>(x)); }
  static AKG_DEV compute load(storage s) { return static_cast<float>(s); }
  static AKG_DEV storage store(compute x) { return static_cast<half_t>(x); }
};
struct bf16 {
  typedef bfloat_t storage;
  typedef float compute;
  static AKG_DEV compute rnd(compute x) { return static_cast<float>(static_cast<bfloat_t>(x)); }
  static AKG_DEV compute load(storage s) { return static_cast<float>(s); }
  static AKG_DEV storage store(compute x) { return static_cast<bfloat_t>(x); }
};
struct i8 {
  typedef s8 storage;
  typedef int compute;
  static AKG_DEV compute rnd(compute x) { return static_cast<int>(static_cast<s8>(x)); }
  static AKG_DEV compute load(storage s) { return static_cast<int>(s); }
  static AKG_DEV storage store(compute x) { return static_cast<s8>(x); }
};
struct i16 {
  typedef short storage;
  typedef int compute;
  static AKG_DEV compute rnd(compute x) { return static_cast<int>(static_cast<short>(x)); }
  static AKG_DEV compute load(storage s) { return static_cast<int>(s); }
  static AKG_DEV storage store(compute x) { return static_cast<short>(x); }
};
struct i32 {
  typedef int storage;
  typedef int compute;
  static AKG_DEV compute rnd(compute x) { return x; }
  static AKG_DEV compute load(storage s) { return s; }
  static AKG_DEV storage store(compute x) { return x; }
};
struct i64 {
  typedef long long storage;
  typedef long long compute;
  static AKG_DEV compute rnd(compute x) { return x; }
  static AKG_DEV compute load(storage s) { return s; }
  static AKG_DEV storage store(compute x) { return x; }
};
// i1 tensors live in memory as one byte per element (0 or 1).
struct b1 {
  typedef u8 storage;
  typedef bool compute;
  static AKG_DEV compute rnd(compute x) { return x; }
  static AKG_DEV compute load(storage s) { return s != 0; }
  static AKG_DEV storage store(compute x) { return x ? 1 : 0; }
};

template <typename T>
struct is_float_compute {
  static constexpr bool value = false;
};
template <>
struct is_float_compute<float> {
  static constexpr bool value = true;
};
template <>
struct is_float_compute<double> {
  static constexpr bool value = true;
};

// ---------------------------------------------------------------------------------------------------------
// Vector memory access. A chunk of V consecutive elements is moved with the widest instructions the
// alignment allows (the lowering only picks V such that every chunk start is V-element aligned).
// ---------------------------------------------------------------------------------------------------------
// Raw register image of a piece of a chunk: at most 16 bytes per memory instruction.
template <int BYTES>
struct Raw;
template <>
struct Raw<16> {
  typedef u32 __attribute__((ext_vector_type(4))) type;
};
template <>
struct Raw<8> {
  typedef u32 __attribute__((ext_vector_type(2))) type;
};
template <>
struct Raw<4> {
  typedef u32 type;
};
template <>
struct Raw<2> {
  typedef u16 type;
};
template <>
struct Raw<1> {
  typedef u8 type;
};

// NT = true marks data that is touched exactly once by the whole grid (streamed tensors): the access is issued
// as a non-temporal one so it does not displace reusable lines (broadcast vectors) from the caches. On MI355X a
// streaming copy gains about 5 % of HBM bandwidth from this.
template <typename DT, int V, bool NT = false>
AKG_DEV void load_chunk(const typename DT::storage *__restrict__ p, typename DT::compute (&dst)[V]) {
  typedef typename DT::storage S;
  constexpr int kBytes = static_cast<int>(sizeof(S)) * V;
  constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  constexpr int kPieces = kBytes / kPiece;
  typedef typename Raw<kPiece>::type R;
  R raw[kPieces];
  const R *rp = reinterpret_cast<const R *>(p);
#pragma unroll
  for (int k = 0; k < kPieces; ++k) raw[k] = NT ? __builtin_nontemporal_load(rp + k) : rp[k];
  S tmp[V];
  __builtin_memcpy(tmp, raw, kBytes);
#pragma unroll
  for (int e = 0; e < V; ++e) dst[e] = DT::load(tmp[e]);
}

template <typename DT, int V, bool NT = false>
AKG_DEV void store_chunk(typename DT::storage *__restrict__ p, const typename DT::compute (&src)[V]) {
  typedef typename DT::storage S;
  constexpr int kBytes = static_cast<int>(sizeof(S)) * V;
  constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  constexpr int kPieces = kBytes / kPiece;
  typedef typename Raw<kPiece>::type R;
  S tmp[V];
#pragma unroll
  for (int e = 0; e < V; ++e) tmp[e] = DT::store(src[e]);
  R raw[kPieces];
  __builtin_memcpy(raw, tmp, kBytes);
  R *rp = reinterpret_cast<R *>(p);
#pragma unroll
  for (int k = 0; k < kPieces; ++k) {
    if (NT) {
      __builtin_nontemporal_store(raw[k], rp + k);
    } else {
      rp[k] = raw[k];
    }
  }
}

// Chunks that are only element-aligned (a slice that starts at an odd column, rows that are not a multiple of the
// chunk): gfx950 serves unaligned 16-byte global accesses, and with the alignment stated truthfully the compiler still
// issues one wide instruction.
template <typename DT, int V>
AKG_DEV void load_chunk_unaligned(const typename DT::storage *__restrict__ p, typename DT::compute (&dst)[V]) {
  typename DT::storage tmp[V];
  __builtin_memcpy(tmp, p, sizeof(tmp));
#pragma unroll
  for (int e = 0; e < V; ++e) dst[e] = DT::load(tmp[e]);
}

template <typename DT, int V>
AKG_DEV void store_chunk_unaligned(typename DT::storage *__restrict__ p, const typename DT::compute (&src)[V]) {
  typename DT::storage tmp[V];
#pragma unroll
  for (int e = 0; e < V; ++e) tmp[e] = DT::store(src[e]);
  __builtin_memcpy(p, tmp, sizeof(tmp));
}

// ---------------------------------------------------------------------------------------------------------
// Buffer-addressed variants (tensors below 2 GiB): a 128-bit descriptor per tensor plus a 32-bit byte offset per
// access, so address arithmetic is 32-bit, and the cache policy of every access is explicit:
//   streamed loads   nt            (touched once: do not keep)
//   streamed stores  sc1 + nt      (write through; measured +2 % over nt alone on a 1 GiB copy)
//   reused loads     default
// ---------------------------------------------------------------------------------------------------------
typedef __amdgpu_buffer_rsrc_t Buffer;

AKG_DEV Buffer make_buffer(const void *p, long bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, static_cast<int>(bytes), 0x00020000);
}

constexpr int kAuxDefault = 0;
constexpr int kAuxStreamLoad = 2;    // nt
#ifndef AKG_STREAM_STORE_AUX
#define AKG_STREAM_STORE_AUX 18
#endif
constexpr int kAuxStreamStore = AKG_STREAM_STORE_AUX;  // sc1 | nt

template <int BYTES, int AUX>
struct BufferIo;
template <int AUX>
struct BufferIo<16, AUX> {
  typedef u32 __attribute__((ext_vector_type(4))) type;
  static AKG_DEV type load(Buffer b, u32 off) { return __builtin_amdgcn_raw_buffer_load_b128(b, off, 0, AUX); }
  static AKG_DEV void store(type v, Buffer b, u32 off) { __builtin_amdgcn_raw_buffer_store_b128(v, b, off, 0, AUX); }
};
template <int AUX>
struct BufferIo<8, AUX> {
  typedef u32 __attribute__((ext_vector_type(2))) type;
  static AKG_DEV type load(Buffer b, u32 off) { return __builtin_amdgcn_raw_buffer_load_b64(b, off, 0, AUX); }
  static AKG_DEV void store(type v, Buffer b, u32 off) { __builtin_amdgcn_raw_buffer_store_b64(v, b, off, 0, AUX); }
};
template <int AUX>
struct BufferIo<4, AUX> {
  typedef u32 type;
  static AKG_DEV type load(Buffer b, u32 off) { return __builtin_amdgcn_raw_buffer_load_b32(b, off, 0, AUX); }
  static AKG_DEV void store(type v, Buffer b, u32 off) { __builtin_amdgcn_raw_buffer_store_b32(v, b, off, 0, AUX); }
};
template <int AUX>
struct BufferIo<2, AUX> {
  typedef u16 type;
  static AKG_DEV type load(Buffer b, u32 off) { return __builtin_amdgcn_raw_buffer_load_b16(b, off, 0, AUX); }
  static AKG_DEV void store(type v, Buffer b, u32 off) { __builtin_amdgcn_raw_buffer_store_b16(v, b, off, 0, AUX); }
};
template <int AUX>
struct BufferIo<1, AUX> {
  typedef u8 type;
  static AKG_DEV type load(Buffer b, u32 off) { return __builtin_amdgcn_raw_buffer_load_b8(b, off, 0, AUX); }
  static AKG_DEV void store(type v, Buffer b, u32 off) { __builtin_amdgcn_raw_buffer_store_b8(v, b, off, 0, AUX); }
};

// `index` is an element index; the chunk starts at byte index * sizeof(storage).
template <typename DT, int V, bool STREAM = false>
AKG_DEV void load_chunk(Buffer buf, long index, typename DT::compute (&dst)[V]) {
  typedef typename DT::storage S;
  constexpr int kBytes = static_cast<int>(sizeof(S)) * V;
  constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  constexpr int kPieces = kBytes / kPiece;
  typedef BufferIo<kPiece, STREAM ? kAuxStreamLoad : kAuxDefault> Io;
  typename Io::type raw[kPieces];
  const u32 off = static_cast<u32>(index) * static_cast<u32>(sizeof(S));
#pragma unroll
  for (int k = 0; k < kPieces; ++k) raw[k] = Io::load(buf, off + k * kPiece);
  S tmp[V];
  __builtin_memcpy(tmp, raw, kBytes);
#pragma unroll
  for (int e = 0; e < V; ++e) dst[e] = DT::load(tmp[e]);
}

template <typename DT, int V, bool STREAM = false>
AKG_DEV void store_chunk(Buffer buf, long index, const typename DT::compute (&src)[V]) {
  typedef typename DT::storage S;
  constexpr int kBytes = static_cast<int>(sizeof(S)) * V;
  constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  constexpr int kPieces = kBytes / kPiece;
  typedef BufferIo<kPiece, STREAM ? kAuxStreamStore : kAuxDefault> Io;
  S tmp[V];
#pragma unroll
  for (int e = 0; e < V; ++e) tmp[e] = DT::store(src[e]);
  typename Io::type raw[kPieces];
  __builtin_memcpy(raw, tmp, kBytes);
  const u32 off = static_cast<u32>(index) * static_cast<u32>(sizeof(S));
#pragma unroll
  for (int k = 0; k < kPieces; ++k) Io::store(raw[k], buf, off + k * kPiece);
}

// The same under a condition that is a value, not a branch: where `ok` is false the access goes to byte 2^31, beyond
// the end of every tensor addressed through a descriptor (they are below 2 GiB), and the range check of the hardware
// answers a load with zeros and drops a store. The accesses of a thread's chunks then issue back to back whatever
// their conditions are, where a branch per chunk would put each behind the test of its own condition.
constexpr u32 kBeyondEveryBuffer = 0x80000000u;

template <typename DT, int V, bool STREAM = false>
AKG_DEV void load_chunk_if(Buffer buf, bool ok, long index, typename DT::compute (&dst)[V]) {
  typedef typename DT::storage S;
  constexpr int kBytes = static_cast<int>(sizeof(S)) * V;
  constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  constexpr int kPieces = kBytes / kPiece;
  typedef BufferIo<kPiece, STREAM ? kAuxStreamLoad : kAuxDefault> Io;
  typename Io::type raw[kPieces];
  const u32 off = ok ? static_cast<u32>(index) * static_cast<u32>(sizeof(S)) : kBeyondEveryBuffer;
#pragma unroll
  for (int k = 0; k < kPieces; ++k) raw[k] = Io::load(buf, off + k * kPiece);
  S tmp[V];
  __builtin_memcpy(tmp, raw, kBytes);
#pragma unroll
  for (int e = 0; e < V; ++e) dst[e] = DT::load(tmp[e]);
}

template <typename DT, int V, bool STREAM = false>
AKG_DEV void store_chunk_if(Buffer buf, bool ok, long index, const typename DT::compute (&src)[V]) {
  typedef typename DT::storage S;
  constexpr int kBytes = static_cast<int>(sizeof(S)) * V;
  constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  constexpr int kPieces = kBytes / kPiece;
  typedef BufferIo<kPiece, STREAM ? kAuxStreamStore : kAuxDefault> Io;
  S tmp[V];
#pragma unroll
  for (int e = 0; e < V; ++e) tmp[e] = DT::store(src[e]);
  typename Io::type raw[kPieces];
  __builtin_memcpy(raw, tmp, kBytes);
  const u32 off = ok ? static_cast<u32>(index) * static_cast<u32>(sizeof(S)) : kBeyondEveryBuffer;
#pragma unroll
  for (int k = 0; k < kPieces; ++k) Io::store(raw[k], buf, off + k * kPiece);
}

// A chunk kept as it came from memory (a 16-bit row held in registers takes half the space of its float image);
// unpack_chunk converts it whenever the values are needed.
template <typename DT, int V>
struct RawChunk {
  static constexpr int kBytes = static_cast<int>(sizeof(typename DT::storage)) * V;
  static constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  static constexpr int kPieces = kBytes / kPiece;
  typename BufferIo<kPiece, kAuxDefault>::type raw[kPieces];
};

template <typename DT, int V, bool STREAM = false>
AKG_DEV void load_raw_chunk(Buffer buf, long index, RawChunk<DT, V> &dst) {
  typedef RawChunk<DT, V> R;
  typedef BufferIo<R::kPiece, STREAM ? kAuxStreamLoad : kAuxDefault> Io;
  const u32 off = static_cast<u32>(index) * static_cast<u32>(sizeof(typename DT::storage));
#pragma unroll
  for (int k = 0; k < R::kPieces; ++k) dst.raw[k] = Io::load(buf, off + k * R::kPiece);
}

template <typename DT, int V, bool STREAM = false>
AKG_DEV void load_raw_chunk_if(Buffer buf, bool ok, long index, RawChunk<DT, V> &dst) {
  typedef RawChunk<DT, V> R;
  typedef BufferIo<R::kPiece, STREAM ? kAuxStreamLoad : kAuxDefault> Io;
  const u32 off = ok ? static_cast<u32>(index) * static_cast<u32>(sizeof(typename DT::storage)) : kBeyondEveryBuffer;
#pragma unroll
  for (int k = 0; k < R::kPieces; ++k) dst.raw[k] = Io::load(buf, off + k * R::kPiece);
}

template <typename DT, int V>
AKG_DEV void zero_raw_chunk(RawChunk<DT, V> &dst) {
#pragma unroll
  for (int k = 0; k < RawChunk<DT, V>::kPieces; ++k) dst.raw[k] = {};
}

// Makes the compiler forget what it knows about the registers of a packed chunk, so that the float values unpacked
// from it in one walk over the row are not kept alive for the next walk (which would defeat the packing).
template <typename DT, int V>
AKG_DEV void forget_unpacked(RawChunk<DT, V> &c) {
#pragma unroll
  for (int k = 0; k < RawChunk<DT, V>::kPieces; ++k) asm volatile("" : "+v"(c.raw[k]));
}

template <typename DT, int V>
AKG_DEV void unpack_chunk(const RawChunk<DT, V> &src, typename DT::compute (&dst)[V]) {
  typename DT::storage tmp[V];
  __builtin_memcpy(tmp, src.raw, RawChunk<DT, V>::kBytes);
#pragma unroll
  for (int e = 0; e < V; ++e) dst[e] = DT::load(tmp[e]);
}

template <typename DT>
AKG_DEV typename DT::compute load_one(Buffer buf, long index) {
  typedef typename DT::storage S;
  typedef BufferIo<static_cast<int>(sizeof(S)), kAuxDefault> Io;
  const typename Io::type raw = Io::load(buf, static_cast<u32>(index) * static_cast<u32>(sizeof(S)));
  S s;
  __builtin_memcpy(&s, &raw, sizeof(S));
  return DT::load(s);
}

template <typename DT>
AKG_DEV void store_one(Buffer buf, long index, typename DT::compute x) {
  typedef typename DT::storage S;
  typedef BufferIo<static_cast<int>(sizeof(S)), kAuxDefault> Io;
  const S s = DT::store(x);
  typename Io::type raw;
  __builtin_memcpy(&raw, &s, sizeof(S));
  Io::store(raw, buf, static_cast<u32>(index) * static_cast<u32>(sizeof(S)));
}

// Workgroups are handed to the 8 XCDs round robin (workgroup w runs on XCD w % 8), and every XCD has an L2 of its own.
// When neighbouring workgroups write parts of the same cache line (rows that are not a multiple of the line), the two
// parts end up in two L2s and reach memory as two partial writes. This renumbering gives every XCD one contiguous
// range of the logical workgroup ids instead, so that neighbours share an L2: XCD x owns grid / 8 ids (one more for
// the first grid % 8 XCDs), in launch order.
AKG_DEV int xcd_contiguous_id(int w, int grid) {
  const int q = grid / 8, r = grid % 8, x = w % 8;
  return x * q + (x < r ? x : r) + w / 8;
}

template <typename DT, int V>
AKG_DEV void fill_chunk(typename DT::compute (&dst)[V], typename DT::compute x) {
#pragma unroll
  for (int e = 0; e < V; ++e) dst[e] = x;
}

// ---------------------------------------------------------------------------------------------------------
// Scalar op semantics. Overloaded on the compute type; names follow the op vocabulary.
// Float ops are plain IEEE single operations (the build disables contraction), division and square root are
// correctly rounded, transcendental functions are the device math library's.
// ---------------------------------------------------------------------------------------------------------
AKG_DEV float op_add(float a, float b) { return a + b; }
AKG_DEV double op_add(double a, double b) { return a + b; }
AKG_DEV int op_add(int a, int b) { return static_cast<int>(static_cast<u32>(a) + static_cast<u32>(b)); }
AKG_DEV long long op_add(long long a, long long b) { return static_cast<long long>(static_cast<u64>(a) + static_cast<u64>(b)); }

AKG_DEV float op_sub(float a, float b) { return a - b; }
AKG_DEV double op_sub(double a, double b) { return a - b; }
AKG_DEV int op_sub(int a, int b) { return static_cast<int>(static_cast<u32>(a) - static_cast<u32>(b)); }
AKG_DEV long long op_sub(long long a, long long b) { return static_cast<long long>(static_cast<u64>(a) - static_cast<u64>(b)); }

AKG_DEV float op_mul(float a, float b) { return a * b; }
AKG_DEV double op_mul(double a, double b) { return a * b; }
AKG_DEV int op_mul(int a, int b) { return static_cast<int>(static_cast<u32>(a) * static_cast<u32>(b)); }
AKG_DEV long long op_mul(long long a, long long b) { return static_cast<long long>(static_cast<u64>(a) * static_cast<u64>(b)); }

AKG_DEV float op_div(float a, float b) { return a / b; }
AKG_DEV double op_div(double a, double b) { return a / b; }
// arith.divsi; a zero divisor is undefined there and yields 0 here.
AKG_DEV int op_div(int a, int b) { return b == 0 ? 0 : ((a == (-2147483647 - 1) && b == -1) ? a : a / b); }
AKG_DEV long long op_div(long long a, long long b) { return b == 0 ? 0 : ((b == -1) ? static_cast<long long>(0ull - static_cast<u64>(a)) : a / b); }

AKG_DEV float op_neg(float a) { return -a; }
AKG_DEV double op_neg(double a) { return -a; }
AKG_DEV int op_neg(int a) { return static_cast<int>(0u - static_cast<u32>(a)); }
AKG_DEV long long op_neg(long long a) { return static_cast<long long>(0ull - static_cast<u64>(a)); }

AKG_DEV float op_abs(float a) { return __builtin_fabsf(a); }
AKG_DEV double op_abs(double a) { return __builtin_fabs(a); }
AKG_DEV int op_abs(int a) { return a < 0 ? op_neg(a) : a; }
AKG_DEV long long op_abs(long long a) { return a < 0 ? op_neg(a) : a; }

// arith.maximumf / arith.minimumf: NaN-propagating.
AKG_DEV float op_maximum(float a, float b) { return (a != a) ? a : ((b != b) ? b : __builtin_fmaxf(a, b)); }
AKG_DEV double op_maximum(double a, double b) { return (a != a) ? a : ((b != b) ? b : __builtin_fmax(a, b)); }
AKG_DEV int op_maximum(int a, int b) { return a > b ? a : b; }
AKG_DEV long long op_maximum(long long a, long long b) { return a > b ? a : b; }
AKG_DEV float op_minimum(float a, float b) { return (a != a) ? a : ((b != b) ? b : __builtin_fminf(a, b)); }
AKG_DEV double op_minimum(double a, double b) { return (a != a) ? a : ((b != b) ? b : __builtin_fmin(a, b)); }
AKG_DEV int op_minimum(int a, int b) { return a < b ? a : b; }
AKG_DEV long long op_minimum(long long a, long long b) { return a < b ? a : b; }

AKG_DEV float op_exp(float a) { return expf(a); }
AKG_DEV double op_exp(double a) { return exp(a); }
AKG_DEV float op_log(float a) { return logf(a); }
AKG_DEV double op_log(double a) { return log(a); }
// float32 tanh, maximum relative error about 1e-6 (the bar for float32 results is 1e-5 against libm):
//   |a| <  0.25 : a * (1 + a^2 * Q(a^2)), the odd Taylor series through a^9 (truncation below 1e-8 relative); the
//                 product form keeps the sign of a zero argument, as libm's tanhf does
//   |a| >= 0.25 : 1 - 2 / (exp(2|a|) + 1) with the hardware exp2 and reciprocal (1 ulp each); the subtraction
//                 loses at most log2(1 / tanh(0.25)) = 2 bits there
// A third of the instructions of the device library's tanhf, which a 64 MiB elementwise kernel cannot hide.
AKG_DEV float op_tanh(float a) {
  const float ax = __builtin_fabsf(a);
  const float z = a * a;
  float q = __builtin_fmaf(0x1.664f48p-6f, z, -0x1.ba1ba2p-5f);  // 62/2835, -17/315
  q = __builtin_fmaf(q, z, 0x1.111112p-3f);                       // 2/15
  q = __builtin_fmaf(q, z, -0x1.555556p-2f);                      // -1/3
  const float small = a * __builtin_fmaf(z, q, 1.0f);
  const float t = __builtin_amdgcn_exp2f(ax * 0x1.715476p+1f);    // exp(2|a|); +inf beyond |a| = 44.4
  const float big = __builtin_fmaf(-2.0f, __builtin_amdgcn_rcpf(t + 1.0f), 1.0f);
  return (ax < 0.25f) ? small : __builtin_copysignf(big, a);      // NaN takes the second branch and stays NaN
}
AKG_DEV double op_tanh(double a) { return tanh(a); }
AKG_DEV float op_sqrt(float a) { return __builtin_sqrtf(a); }
AKG_DEV double op_sqrt(double a) { return __builtin_sqrt(a); }
// math.rsqrt reaches the CPU as 1 / sqrt(x): two correctly rounded operations.
AKG_DEV float op_rsqrt(float a) { return 1.0f / __builtin_sqrtf(a); }
AKG_DEV double op_rsqrt(double a) { return 1.0 / __builtin_sqrt(a); }
AKG_DEV float op_inv(float a) { return 1.0f / a; }
AKG_DEV double op_inv(double a) { return 1.0 / a; }
AKG_DEV float op_floor(float a) { return __builtin_floorf(a); }
AKG_DEV double op_floor(double a) { return __builtin_floor(a); }
AKG_DEV float op_sin(float a) { return sinf(a); }
AKG_DEV double op_sin(double a) { return sin(a); }
AKG_DEV float op_cos(float a) { return cosf(a); }
AKG_DEV double op_cos(double a) { return cos(a); }
AKG_DEV float op_asin(float a) { return asinf(a); }
AKG_DEV double op_asin(double a) { return asin(a); }
AKG_DEV float op_acos(float a) { return acosf(a); }
AKG_DEV double op_acos(double a) { return acos(a); }
AKG_DEV float op_atan(float a) { return atanf(a); }
AKG_DEV double op_atan(double a) { return atan(a); }
AKG_DEV float op_pow(float a, float b) { return powf(a, b); }
AKG_DEV double op_pow(double a, double b) { return pow(a, b); }
AKG_DEV float op_atan2(float a, float b) { return atan2f(a, b); }
AKG_DEV double op_atan2(double a, double b) { return atan2(a, b); }

AKG_DEV bool op_isnan(float a) { return a != a; }
AKG_DEV bool op_isnan(double a) { return a != a; }
AKG_DEV bool op_isinf(float a) { return __builtin_fabsf(a) == __builtin_inff(); }
AKG_DEV bool op_isinf(double a) { return __builtin_fabs(a) == __builtin_inf(); }
AKG_DEV bool op_isfinite(float a) { return __builtin_fabsf(a) < __builtin_inff(); }
AKG_DEV bool op_isfinite(double a) { return __builtin_fabs(a) < __builtin_inf(); }

// ---------------------------------------------------------------------------------------------------------
// Exact float32 division by a value that is the same for a whole row (softmax denominators, quantisation
// scales). The correctly rounded reciprocal is computed once per row; per element the quotient is
// q = a * rcp followed by one FMA residual correction, which yields the correctly rounded a / b (Markstein)
// as long as nothing under- or overflows on the way. Operands outside a conservative exponent window, and
// zero dividends (whose sign the correction would lose), take the ordinary IEEE division instead.
// ---------------------------------------------------------------------------------------------------------
struct UniformDivisor {
  float b;
  float rcp;
  bool safe;
};
AKG_DEV UniformDivisor make_divisor(float b) {
  UniformDivisor d;
  d.b = b;
  d.rcp = 1.0f / b;
  const float ab = __builtin_fabsf(b);
  d.safe = (ab >= 0x1p-60f) && (ab <= 0x1p+60f);
  return d;
}
AKG_DEV float div_uniform(float a, const UniformDivisor &d) {
  const float aa = __builtin_fabsf(a);
  const bool fast = d.safe && (aa >= 0x1p-60f) && (aa <= 0x1p+60f);
  const float q = a * d.rcp;
  const float rem = __builtin_fmaf(-q, d.b, a);
  float res = __builtin_fmaf(rem, d.rcp, q);
  if (__builtin_expect(!fast, 0)) res = a / d.b;
  return res;
}

// ---------------------------------------------------------------------------------------------------------
// Relaxed math, used only for values whose every path to a kernel output passes through a cast to a 16-bit
// float (11 or 8 significant bits): hardware transcendental instructions (about 1 ulp of float32) instead of
// the correctly rounded / libm-grade sequences. Never used on paths that reach a float32 or integer output.
// ---------------------------------------------------------------------------------------------------------
AKG_DEV float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
AKG_DEV float fast_div(float a, float b) { return a * __builtin_amdgcn_rcpf(b); }
AKG_DEV float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 0x1.715476p+0f); }
AKG_DEV float fast_log(float x) { return __builtin_amdgcn_logf(x) * 0x1.62e43p-1f; }
AKG_DEV float fast_sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
AKG_DEV float fast_rsqrt(float x) { return __builtin_amdgcn_rsqf(x); }
AKG_DEV float fast_tanh(float x) {
  // tanh(x) = 1 - 2 / (exp(2x) + 1): exp overflow gives 1, underflow gives -1. Near zero the subtraction cancels, so
  // the absolute error stays about 1e-7 while the relative error grows; values that need more never get here.
  const float t = __builtin_amdgcn_exp2f(x * 0x1.715476p+1f);
  return __builtin_fmaf(-2.0f, __builtin_amdgcn_rcpf(t + 1.0f), 1.0f);
}

// Reduction combiners (arith.addf / maxnumf / minnumf / mulf and their integer twins).
struct RedSum {
  template <typename T>
  static AKG_DEV T apply(T a, T b) { return op_add(a, b); }
};
struct RedProd {
  template <typename T>
  static AKG_DEV T apply(T a, T b) { return op_mul(a, b); }
};
struct RedMax {
  static AKG_DEV float apply(float a, float b) { return __builtin_fmaxf(a, b); }
  static AKG_DEV double apply(double a, double b) { return __builtin_fmax(a, b); }
  static AKG_DEV int apply(int a, int b) { return a > b ? a : b; }
  static AKG_DEV long long apply(long long a, long long b) { return a > b ? a : b; }
};
struct RedMin {
  static AKG_DEV float apply(float a, float b) { return __builtin_fminf(a, b); }
  static AKG_DEV double apply(double a, double b) { return __builtin_fmin(a, b); }
  static AKG_DEV int apply(int a, int b) { return a < b ? a : b; }
  static AKG_DEV long long apply(long long a, long long b) { return a < b ? a : b; }
};
struct RedAll {
  static AKG_DEV bool apply(bool a, bool b) { return a && b; }
};
struct RedAny {
  static AKG_DEV bool apply(bool a, bool b) { return a || b; }
};

// ---------------------------------------------------------------------------------------------------------
// Cast (tosa.cast): float->float rounds to nearest even; float->int rounds to nearest even, saturates to the
// destination range, then converts; float->bool is `!= 0`; int->float converts exactly or to nearest even;
// int->narrower int saturates; int->bool is `!= 0`.
// ---------------------------------------------------------------------------------------------------------
template <typename DST>
struct IntRange;
template <>
struct IntRange<i8> {
  static constexpr long long lo = -128, hi = 127;
};
template <>
struct IntRange<i16> {
  static constexpr long long lo = -32768, hi = 32767;
};
template <>
struct IntRange<i32> {
  static constexpr long long lo = -2147483648LL, hi = 2147483647LL;
};
template <>
struct IntRange<i64> {
  static constexpr long long lo = (-9223372036854775807LL - 1), hi = 9223372036854775807LL;
};

template <typename DST, typename SRC>
struct Caster {
  // float -> float, int -> float (compute types are convertible; rnd applies the destination precision)
  static AKG_DEV typename DST::compute run(typename SRC::compute x) {
    return DST::rnd(static_cast<typename DST::compute>(x));
  }
};

// math.roundeven
AKG_DEV float round_even(float x) { return __builtin_rintf(x); }
AKG_DEV double round_even(double x) { return __builtin_rint(x); }

template <typename DST, typename SRCC, bool SrcIsFloat>
struct ToInt;
template <typename DST, typename SRCC>
struct ToInt<DST, SRCC, true> {
  static AKG_DEV typename DST::compute run(SRCC x) {
    SRCC r = round_even(x);
    const SRCC lo = static_cast<SRCC>(IntRange<DST>::lo);
    const SRCC hi = static_cast<SRCC>(IntRange<DST>::hi);
    if (r != r) return 0;
    if (r <= lo) return static_cast<typename DST::compute>(IntRange<DST>::lo);
    if (r >= hi) return static_cast<typename DST::compute>(IntRange<DST>::hi);
    return static_cast<typename DST::compute>(r);
  }
};
// float32 -> int8 / int16: both bounds are float32 values, so the clamp is one v_med3_f32 and the conversion is
// always in range: v_rndne_f32, v_med3_f32, v_cvt_i32_f32 (+ the NaN -> 0 select).
template <>
struct ToInt<i8, float, true> {
  static AKG_DEV int run(float x) {
    float r = __builtin_amdgcn_fmed3f(__builtin_rintf(x), -128.0f, 127.0f);
    return (x != x) ? 0 : static_cast<int>(r);
  }
};
template <>
struct ToInt<i16, float, true> {
  static AKG_DEV int run(float x) {
    float r = __builtin_amdgcn_fmed3f(__builtin_rintf(x), -32768.0f, 32767.0f);
    return (x != x) ? 0 : static_cast<int>(r);
  }
};
template <typename DST, typename SRCC>
struct ToInt<DST, SRCC, false> {
  static AKG_DEV typename DST::compute run(SRCC x) {
    long long v = static_cast<long long>(x);
    if (v < IntRange<DST>::lo) v = IntRange<DST>::lo;
    if (v > IntRange<DST>::hi) v = IntRange<DST>::hi;
    return static_cast<typename DST::compute>(v);
  }
};

#define AKG_CAST_TO_INT(DSTT)                                                                              \
  template <typename SRC>                                                                                  \
  struct Caster<DSTT, SRC> {                                                                               \
    static AKG_DEV typename DSTT::compute run(typename SRC::compute x) {                                   \
      return ToInt<DSTT, typename SRC::compute, is_float_compute<typename SRC::compute>::value>::run(x);   \
    }                                                                                                      \
  };
AKG_CAST_TO_INT(i8)
AKG_CAST_TO_INT(i16)
AKG_CAST_TO_INT(i32)
AKG_CAST_TO_INT(i64)
#undef AKG_CAST_TO_INT

template <typename SRC>
struct Caster<b1, SRC> {
  static AKG_DEV bool run(typename SRC::compute x) { return x != static_cast<typename SRC::compute>(0); }
};
// bool sources: 0 / 1 (uitofp / zext)
template <typename DST>
struct FromBool {
  static AKG_DEV typename DST::compute run(bool x) {
    return x ? static_cast<typename DST::compute>(1) : static_cast<typename DST::compute>(0);
  }
};
template <>
struct Caster<f32, b1> : FromBool<f32> {};
template <>
struct Caster<f64, b1> : FromBool<f64> {};
template <>
struct Caster<f16, b1> : FromBool<f16> {};
template <>
struct Caster<bf16, b1> : FromBool<bf16> {};
template <>
struct Caster<i8, b1> : FromBool<i8> {};
template <>
struct Caster<i16, b1> : FromBool<i16> {};
template <>
struct Caster<i32, b1> : FromBool<i32> {};
template <>
struct Caster<i64, b1> : FromBool<i64> {};
template <>
struct Caster<b1, b1> {
  static AKG_DEV bool run(bool x) { return x; }
};

// Fused clamp + float->int cast: cast(min(max(x, lo), hi)) with constant bounds. Rounding to nearest even is monotonic
// and maps the bounds to integers, so rounding first and clamping to the rounded bounds (already intersected with the
// destination range by the lowering) is the same function; NaN propagates through min/max and casts to 0.
AKG_DEV int clamp_cast(float x, float lo, float hi) {
  const float r = __builtin_amdgcn_fmed3f(__builtin_rintf(x), lo, hi);
  return (x != x) ? 0 : static_cast<int>(r);
}

template <typename DST, typename SRC>
AKG_DEV typename DST::compute cast(typename SRC::compute x) {
  return Caster<DST, SRC>::run(x);
}

// ---------------------------------------------------------------------------------------------------------
// Cross-lane reductions. A row is owned by a group of TPR threads (TPR a power of two). Up to one wavefront
// the reduction is a butterfly of pairwise exchanges: at every step each lane combines its partial result with
// the partial result of exactly one partner group, and both partners combine the same two values, so every lane
// ends with the same bits. No step goes through LDS:
//   partner distance 1, 2   DPP quad_perm
//   4                       DPP row_half_mirror (lane i <-> 7 - i of its 8-lane half row: the other quad)
//   8                       DPP row_mirror      (lane i <-> 15 - i of its 16-lane row: the other half row)
//   16                      v_permlane16_swap   (exchanges odd and even 16-lane rows)
//   32                      v_permlane32_swap   (exchanges the two 32-lane halves)
// Groups wider than a wavefront finish through a small LDS array; every thread then folds the per-wavefront
// partials in the same fixed order.
// ---------------------------------------------------------------------------------------------------------
template <int STEP>
AKG_DEV u32 lane_partner_bits(u32 v) {
  if constexpr (STEP == 1) {
    return static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, true));  // [1,0,3,2]
  } else if constexpr (STEP == 2) {
    return static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, true));  // [2,3,0,1]
  } else if constexpr (STEP == 4) {
    return static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x141, 0xF, 0xF, true));
  } else if constexpr (STEP == 8) {
    return static_cast<u32>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x140, 0xF, 0xF, true));
  } else if constexpr (STEP == 16) {
    // result[0] keeps this lane's value in even rows and receives the partner's in odd rows; result[1] the reverse
    const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    return r[0] ^ r[1] ^ v;
  } else {
    static_assert(STEP == 32, "partner distance must be a power of two up to 32");
    const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return r[0] ^ r[1] ^ v;
  }
}

template <int STEP>
AKG_DEV float lane_partner(float v) {
  return __builtin_bit_cast(float, lane_partner_bits<STEP>(__builtin_bit_cast(u32, v)));
}
template <int STEP>
AKG_DEV int lane_partner(int v) {
  return static_cast<int>(lane_partner_bits<STEP>(static_cast<u32>(v)));
}
template <int STEP>
AKG_DEV bool lane_partner(bool v) {
  return lane_partner_bits<STEP>(v ? 1u : 0u) != 0u;
}
template <int STEP>
AKG_DEV double lane_partner(double v) {
  const u64 b = __builtin_bit_cast(u64, v);
  const u32 lo = lane_partner_bits<STEP>(static_cast<u32>(b & 0xffffffffu));
  const u32 hi = lane_partner_bits<STEP>(static_cast<u32>(b >> 32));
  return __builtin_bit_cast(double, (static_cast<u64>(hi) << 32) | lo);
}
template <int STEP>
AKG_DEV long long lane_partner(long long v) {
  const u64 b = static_cast<u64>(v);
  const u32 lo = lane_partner_bits<STEP>(static_cast<u32>(b & 0xffffffffu));
  const u32 hi = lane_partner_bits<STEP>(static_cast<u32>(b >> 32));
  return static_cast<long long>((static_cast<u64>(hi) << 32) | lo);
}

template <typename Red, int WIDTH, typename T>
AKG_DEV T wave_group_reduce(T v) {
  static_assert(WIDTH <= kWaveSize && (WIDTH & (WIDTH - 1)) == 0, "group width must be a power of two <= 64");
  if constexpr (WIDTH > 1) v = Red::apply(v, lane_partner<1>(v));
  if constexpr (WIDTH > 2) v = Red::apply(v, lane_partner<2>(v));
  if constexpr (WIDTH > 4) v = Red::apply(v, lane_partner<4>(v));
  if constexpr (WIDTH > 8) v = Red::apply(v, lane_partner<8>(v));
  if constexpr (WIDTH > 16) v = Red::apply(v, lane_partner<16>(v));
  if constexpr (WIDTH > 32) v = Red::apply(v, lane_partner<32>(v));
  return v;
}

// Reduction over a group of TPR threads. `scratch` points at this reduction's LDS slots (one per wavefront of
// the block); it is only touched when TPR > 64. The caller alternates between two scratch arrays from one
// reduction to the next, which makes a single barrier per reduction sufficient.
template <typename Red, int TPR, typename T>
AKG_DEV T group_reduce(T v, T *scratch, int tid) {
  if constexpr (TPR <= kWaveSize) {
    return wave_group_reduce<Red, TPR>(v);
  } else {
    constexpr int kWavesPerGroup = TPR / kWaveSize;
    v = wave_group_reduce<Red, kWaveSize>(v);
    const int wave = tid / kWaveSize;
    if ((tid % kWaveSize) == 0) scratch[wave] = v;
    __syncthreads();
    const int first = (wave / kWavesPerGroup) * kWavesPerGroup;
    T r = scratch[first];
#pragma unroll
    for (int w = 1; w < kWavesPerGroup; ++w) r = Red::apply(r, scratch[first + w]);
    return r;
  }
}

// ---------------------------------------------------------------------------------------------------------
// Column kernels: a chunk of V columns kept as it came from memory, and reductions whose V lanes are V different runs.
// ---------------------------------------------------------------------------------------------------------
template <typename DT, int V>
struct PackedChunk {
  static constexpr int kBytes = static_cast<int>(sizeof(typename DT::storage)) * V;
  static_assert(kBytes <= 16, "a packed chunk is one memory access");
  typename Raw<kBytes>::type raw;
};

template <typename DT, int V, bool NT = false>
AKG_DEV void load_packed(const typename DT::storage *__restrict__ p, PackedChunk<DT, V> &dst) {
  typedef typename Raw<PackedChunk<DT, V>::kBytes>::type R;
  const R *rp = reinterpret_cast<const R *>(p);
  dst.raw = NT ? __builtin_nontemporal_load(rp) : *rp;
}

template <typename DT, int V>
AKG_DEV void zero_packed(PackedChunk<DT, V> &dst) {
  dst.raw = {};
}

// The first n elements of a chunk that is only element-aligned (n = V: one unaligned access); the rest is zero.
template <typename DT, int V>
AKG_DEV void load_packed_partial(const typename DT::storage *__restrict__ p, int n, PackedChunk<DT, V> &dst) {
  typename DT::storage tmp[V];
  if (n == V) {
    __builtin_memcpy(tmp, p, sizeof(tmp));
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) tmp[e] = e < n ? p[e] : typename DT::storage();
  }
  __builtin_memcpy(&dst.raw, tmp, sizeof(tmp));
}

// Makes the compiler forget what it derived from a resident chunk: the next walk unpacks it again instead of keeping
// every unpacked (or further computed) element of the previous walk alive in registers of its own.
template <typename DT, int V>
AKG_DEV void forget_derived(PackedChunk<DT, V> &p) {
  if constexpr (PackedChunk<DT, V>::kBytes >= 4) asm volatile("" : "+v"(p.raw));
}

template <typename DT, int V>
AKG_DEV void unpack_packed(const PackedChunk<DT, V> &src, typename DT::compute (&dst)[V]) {
  typename DT::storage tmp[V];
  __builtin_memcpy(tmp, &src.raw, sizeof(tmp));
#pragma unroll
  for (int e = 0; e < V; ++e) dst[e] = DT::load(tmp[e]);
}

// The first n elements of a chunk to an address that is only element-aligned.
template <typename DT, int V>
AKG_DEV void store_chunk_partial(typename DT::storage *__restrict__ p, int n, const typename DT::compute (&src)[V]) {
  if (n == V) {
    store_chunk_unaligned<DT, V>(p, src);
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      if (e < n) p[e] = DT::store(src[e]);
    }
  }
}

// Thread tid = ly * LX + lx of a workgroup of BLOCK threads holds V partial results for the columns of lx; on return
// every thread holds the results over all ly. Partners inside a wavefront first (lanes LX, 2 LX, ... apart hold the
// same columns), then the wavefronts through `scratch` ((BLOCK / 64) * LX * V values; the caller alternates between
// two such arrays from one reduction to the next, so one barrier per reduction suffices). ROUND: DT::rnd after every
// step, which keeps a narrow result type's rounding (sums and products; a maximum is one of its operands).
template <typename Red, typename DT, bool ROUND, typename T>
AKG_DEV T column_step(T a, T b) {
  if constexpr (ROUND) {
    return DT::rnd(Red::apply(a, b));
  } else {
    return Red::apply(a, b);
  }
}

template <typename Red, typename DT, bool ROUND, int LX, int BLOCK, int V>
AKG_DEV void column_reduce(typename DT::compute (&acc)[V], typename DT::compute *scratch, int tid) {
  static_assert(LX <= kWaveSize && (LX & (LX - 1)) == 0 && BLOCK % kWaveSize == 0, "column groups are powers of two within a wavefront");
  typedef typename DT::compute T;
#pragma unroll
  for (int e = 0; e < V; ++e) {
    T v = acc[e];
    if constexpr (LX <= 1) v = column_step<Red, DT, ROUND>(v, lane_partner<1>(v));
    if constexpr (LX <= 2) v = column_step<Red, DT, ROUND>(v, lane_partner<2>(v));
    // (lane_partner<4> and <8> mirror their groups, which is no good here: the partner must hold the same columns)
    if constexpr (LX <= 4) v = column_step<Red, DT, ROUND>(v, static_cast<T>(__shfl_xor(v, 4)));
    if constexpr (LX <= 8) v = column_step<Red, DT, ROUND>(v, static_cast<T>(__shfl_xor(v, 8)));
    if constexpr (LX <= 16) v = column_step<Red, DT, ROUND>(v, lane_partner<16>(v));
    if constexpr (LX <= 32) v = column_step<Red, DT, ROUND>(v, lane_partner<32>(v));
    acc[e] = v;
  }
  if constexpr (BLOCK > kWaveSize) {
    constexpr int kWaves = BLOCK / kWaveSize;
    const int wave = tid / kWaveSize, lane = tid % kWaveSize, lx = tid % LX;
    if (lane < LX) {
#pragma unroll
      for (int e = 0; e < V; ++e) scratch[(wave * LX + lx) * V + e] = acc[e];
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < V; ++e) {
      T r = scratch[lx * V + e];
#pragma unroll
      for (int w = 1; w < kWaves; ++w) r = column_step<Red, DT, ROUND>(r, scratch[(w * LX + lx) * V + e]);
      acc[e] = r;
    }
  }
}

// ---------------------------------------------------------------------------------------------------------
// Ordered reductions. A sum or a product whose declared result is float16 / bfloat16 is rounded to that type after
// every step, so the order of the steps is part of the result: the reference runs ONE serial loop per result
// element, in index order (linalg.reduce lowered to loops, MindSporeToLinalg.cpp:845-901,1333-1451). 4096 float16
// ones sum to 2048 that way, and to 4096 in a tree. The kernels keep that order: the elements of a run go through
// LDS in their declared 16-bit type (what they hold is already rounded to it), and one thread per run folds them one
// after the other; many runs fold side by side on the lanes of a wavefront.
// ---------------------------------------------------------------------------------------------------------
// Elements e >= from of a thread's chunk to positions at + e of a run's LDS image.
template <typename DT, int V>
AKG_DEV void chain_put(typename DT::storage *run, int at, const typename DT::compute (&v)[V], int from) {
  static_assert(sizeof(typename DT::storage) == 2, "ordered reductions are those of the 16-bit float types");
  if constexpr (V * 2 >= 4 && V * 2 <= 16) {
    if (from == 0 && (at % V) == 0) {
      typename DT::storage tmp[V];
#pragma unroll
      for (int e = 0; e < V; ++e) tmp[e] = DT::store(v[e]);
      typedef typename Raw<V * 2>::type R;
      R raw;
      __builtin_memcpy(&raw, tmp, sizeof(tmp));
      *reinterpret_cast<R *>(run + at) = raw;
      return;
    }
  }
#pragma unroll
  for (int e = 0; e < V; ++e) {
    if (e >= from) run[at + e] = DT::store(v[e]);
  }
}

// acc folded with run[0 .. n) in index order, rounded to the declared type after every step.
// `run` is 16-byte aligned.
template <typename Red, typename DT>
AKG_DEV typename DT::compute chain_fold(typename DT::compute acc, const typename DT::storage *run, int n) {
  int i = 0;
  for (; i + 8 <= n; i += 8) {
    typename DT::storage tmp[8];
    const typename Raw<16>::type raw = *reinterpret_cast<const typename Raw<16>::type *>(run + i);
    __builtin_memcpy(tmp, &raw, sizeof(tmp));
#pragma unroll
    for (int e = 0; e < 8; ++e) acc = DT::rnd(Red::apply(acc, DT::load(tmp[e])));
  }
  for (; i < n; ++i) acc = DT::rnd(Red::apply(acc, DT::load(run[i])));
  return acc;
}

// Column kernels: thread (ly, lx) of LY x LX holds V values of row `first + ly` of the run, columns lx * V + e. The
// rows of one step are neighbours in the run, so a step puts them into LDS ([LY][LX * V]) and the thread that owns
// column c = tid, tid + BLOCK, ... folds rows 0 .. nrows - 1 of it onto its accumulator, in order.
template <typename Red, typename DT, int LX, int BLOCK, int V, int NOWN>
AKG_DEV void column_chain_step(typename DT::compute (&own)[NOWN], const typename DT::compute (&v)[V],
                               typename DT::storage *lds, int tid, int nrows) {
  constexpr int kCols = LX * V;
  const int lx = tid % LX, ly = tid / LX;
  chain_put<DT, V>(lds + ly * kCols, lx * V, v, 0);
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NOWN; ++k) {
    const int c = tid + k * BLOCK;
    if (c < kCols) {
      typename DT::compute a = own[k];
      for (int r = 0; r < nrows; ++r) a = DT::rnd(Red::apply(a, DT::load(lds[r * kCols + c])));
      own[k] = a;
    }
  }
  __syncthreads();
}

// The owners' results to every thread of the column (`res`: LX * V values of the compute type).
template <typename DT, int LX, int BLOCK, int V, int NOWN>
AKG_DEV void column_chain_finish(const typename DT::compute (&own)[NOWN], typename DT::compute (&acc)[V],
                                 typename DT::compute *res, int tid) {
  constexpr int kCols = LX * V;
#pragma unroll
  for (int k = 0; k < NOWN; ++k) {
    const int c = tid + k * BLOCK;
    if (c < kCols) res[c] = own[k];
  }
  __syncthreads();
  const int lx = tid % LX;
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = res[lx * V + e];
}

// ---------------------------------------------------------------------------------------------------------
// Workspace protocol of the streaming reductions. Several workgroups share one group of outputs; each leaves
// its partial result in device memory and counts its arrival; the workgroup that arrives last reads all the
// partials back (in slot order, so the result does not depend on the arrival order) and finishes the job.
//
// The eight XCDs have private L2 caches. A device-scope release fence per workgroup would write back and an
// acquire fence would invalidate a whole L2 each time (measured: about 1 us per workgroup, serialised per XCD),
// so the protocol uses no fence. Partials are written and read with device-scope (sc1) accesses, which go
// through the L2 to memory and back; a thread waits for its own stores to be acknowledged (vmcnt 0) before the
// workgroup barrier, and one thread then counts the arrival with a device-scope atomic. The last workgroup puts
// the counter back to zero: the workspace is zero-filled once when it is allocated and every launch leaves it
// as it found it.
// ---------------------------------------------------------------------------------------------------------
constexpr int kAuxDeviceScope = 16;  // sc1

template <typename T>
AKG_DEV void ws_store(T *p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
AKG_DEV T ws_load(const T *p) {
  return __hip_atomic_load(const_cast<T *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// V adjacent partials of one lane at byte offset `off` of the workspace (aligned to min(16, V * sizeof(T))).
template <int V, typename T>
AKG_DEV void ws_store_chunk(Buffer ws, u32 off, const T (&v)[V]) {
  constexpr int kBytes = static_cast<int>(sizeof(T)) * V;
  constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  constexpr int kPieces = kBytes / kPiece;
  typedef BufferIo<kPiece, kAuxDeviceScope> Io;
  typename Io::type raw[kPieces];
  __builtin_memcpy(raw, v, kBytes);
#pragma unroll
  for (int k = 0; k < kPieces; ++k) Io::store(raw[k], ws, off + k * kPiece);
}
template <int V, typename T>
AKG_DEV void ws_load_chunk(Buffer ws, u32 off, T (&v)[V]) {
  constexpr int kBytes = static_cast<int>(sizeof(T)) * V;
  constexpr int kPiece = kBytes > 16 ? 16 : kBytes;
  constexpr int kPieces = kBytes / kPiece;
  typedef BufferIo<kPiece, kAuxDeviceScope> Io;
  typename Io::type raw[kPieces];
#pragma unroll
  for (int k = 0; k < kPieces; ++k) raw[k] = Io::load(ws, off + k * kPiece);
  __builtin_memcpy(v, raw, kBytes);
}

// ... or, where `ok` is false, nothing: the load is issued beyond the buffer and leaves zeros (no branch around it, so
// that the loads of a trip go out together).
template <int V, typename T>
AKG_DEV void ws_load_chunk_if(Buffer ws, bool ok, u32 off, T (&v)[V]) {
  ws_load_chunk<V>(ws, ok ? off : kBeyondEveryBuffer, v);
}

// True in every thread of exactly one workgroup out of the `split` that share counter `group`: the last to arrive.
// Must be reached by all threads of the workgroup, after their ws_store / ws_store_chunk calls.
AKG_DEV bool last_workgroup(unsigned *counters, long group, int split, int tid, unsigned *flag) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this thread's partials have reached memory
  __syncthreads();
  if (tid == 0) {
    const unsigned prev = __hip_atomic_fetch_add(counters + group, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = prev == static_cast<unsigned>(split - 1);
    if (last) __hip_atomic_store(counters + group, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last ? 1u : 0u;
  }
  __syncthreads();
  const bool last = *flag != 0u;
  asm volatile("" ::: "memory");  // no access to the partials may be moved above the arrival count
  return last;
}

}  // namespace akg
