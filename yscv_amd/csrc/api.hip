// C ABI of the yscv_hip library (declarations and contracts: include/yscv_hip.h).
#include <vector>

#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

// ---- errors / context ------------------------------------------------------------------
std::string &last_error_slot() {
  static thread_local std::string slot;
  return slot;
}

int32_t set_error(int32_t code, const char *fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  last_error_slot() = buf;
  return code;
}

static std::mutex g_ctx_mutex;
static Context g_ctx;
static bool g_ctx_ready = false;

// Scratch of yscv_hip_int4_matmul_static: device memory that exists from the moment the code object is loaded, so
// that entry point never allocates.  Every GPU holds its own copy at its own address; the name below is only the
// host-side handle of the symbol, the address a kernel can use is looked up once per device in init_context().
static __device__ __align__(256) unsigned char scratch[YSCV_HIP_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices] = {};

int32_t init_context(int device) {
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  if (g_ctx_ready && g_ctx.device == device) return YSCV_HIP_OK;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0)
    return set_error(YSCV_HIP_ERR_NO_DEVICE, "no HIP device visible (%s)", hipGetErrorString(e));
  if (device < 0 || device >= count)
    return set_error(YSCV_HIP_ERR_INVALID_ARG, "device index %d out of range (0..%d)", device, count - 1);
  hipDeviceProp_t prop;
  YSCV_HIP_TRY(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(YSCV_HIP_ERR_NO_DEVICE, "device %d is %s; this library is built for gfx950 only", device,
                     prop.gcnArchName);
  YSCV_HIP_TRY(hipSetDevice(device));
  if (device < kMaxDevices && g_scratch_ptr[device] == nullptr) {
    void *p = nullptr;
    YSCV_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_scratch_ptr[device] = p;
  }
  // Calls without a caller-provided workspace take their scratch from the stream-ordered allocator; keeping freed
  // blocks in its pool makes that a sub-microsecond operation instead of a trip to the driver per call.
  hipMemPool_t pool = nullptr;
  if (hipDeviceGetDefaultMemPool(&pool, device) == hipSuccess && pool != nullptr) {
    uint64_t keep = UINT64_MAX;
    (void)hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &keep);
  }
  (void)hipGetLastError();
  g_ctx.device = device;
  g_ctx.num_cus = prop.multiProcessorCount;
  g_ctx.lds_bytes = (int)prop.sharedMemPerBlock;
  g_ctx.total_mem = prop.totalGlobalMem;
  snprintf(g_ctx.arch, sizeof(g_ctx.arch), "%s", prop.gcnArchName);
  snprintf(g_ctx.name, sizeof(g_ctx.name), "%s", prop.name);
  g_ctx_ready = true;
  return YSCV_HIP_OK;
}

int32_t ensure_context(const Context **out) {
  if (!g_ctx_ready) YSCV_TRY(init_context(0));
  if (out) *out = &g_ctx;
  return YSCV_HIP_OK;
}

void drop_context() {
  std::lock_guard<std::mutex> lock(g_ctx_mutex);
  g_ctx_ready = false;
}

static bool valid_act_dtype(int d) { return d == YSCV_HIP_F32 || d == YSCV_HIP_F16 || d == YSCV_HIP_BF16; }
static size_t dtype_size(int d) { return d == YSCV_HIP_F32 ? 4 : 2; }

// Scratch layout of one int4 call: [xh][xl][row_scale][partial], each part rounded to 256 B.
// A fp16 activation whose row stride already equals the padded K needs no preparation at all, and neither does an
// f32 or bf16 one on its way to the skinny kernel, which normalises (and for f32 splits) it on the fly.
struct Int4Scratch {
  bool direct;       // x is used in place as the fp16 `hi` operand
  bool skinny;
  int split;
  size_t k_pad;
  SkinnyPlan plan;
  size_t xh_bytes, rs_bytes, part_bytes, total;
  size_t opt_bytes;  // behind `total`: the K-split partials of the LDS-ring GEMM (0 when that launch is not split)
};

// f32 activations on the exact-scale route with 16 < m <= this many rows run as 16-row skinny calls
constexpr size_t kChunkedSkinnyMaxRows = 128;

static Int4Scratch int4_scratch_layout(const yscv_hip_int4_weight *w, const void *x, int x_dtype, size_t m,
                                       int force, int num_cus) {
  Int4Scratch L{};
  L.skinny = force == 1 || (force == 0 && m <= 16);
  L.k_pad = w->ktp * 128;
  L.direct = (x_dtype == YSCV_HIP_F16 || L.skinny) && L.k_pad == w->k &&
             (reinterpret_cast<uintptr_t>(x) & 15) == 0;
  L.split = x_dtype == YSCV_HIP_F32 ? 2 : 1;
  if (L.skinny) L.plan = plan_int4_skinny(w, m, L.split, num_cus);
  L.xh_bytes = L.direct ? 0 : round_up(m * L.k_pad * sizeof(_Float16), 256);
  L.rs_bytes = L.direct ? 0 : round_up(m * sizeof(float), 256);
  L.part_bytes = L.skinny ? round_up(L.plan.partial_bytes, 256) : 0;
  L.total = L.xh_bytes * L.split + L.rs_bytes + L.part_bytes;
  // partial sums of whichever kernel takes the rows above 16: the register-resident one up to 32 rows where its
  // parts fit the cap, else the LDS-ring GEMM's K split
  if (L.skinny) {
    L.opt_bytes = 0;
  } else if (m <= 32 && int4_mid_partial_bytes(w, m) <= kMidPartialCap) {
    const size_t ring = int4_gemm_ring_partial_bytes(w, m, num_cus);  // the ring takes over if the mid kernel cannot (alignment)
    const size_t mid = int4_mid_partial_bytes(w, m);
    L.opt_bytes = round_up(mid > ring ? mid : ring, 256);
  } else {
    L.opt_bytes = round_up(int4_gemm_ring_partial_bytes(w, m, num_cus), 256);
  }
  if (!L.skinny && force == 0 && x_dtype == YSCV_HIP_F32 && m <= kChunkedSkinnyMaxRows) {
    // this call may run as 16-row skinny calls (see int4_run_ws): the scratch must cover one of those too
    const Int4Scratch c = int4_scratch_layout(w, x, x_dtype, 16, 1, num_cus);
    if (c.total > L.total) L.total = c.total;
  }
  return L;
}

int32_t int4_workspace_bytes(const yscv_hip_int4_weight *w, size_t m, int x_dtype, int force, size_t *bytes) {
  const Context *ctx = nullptr;
  YSCV_TRY(ensure_context(&ctx));
  YSCV_REQUIRE(w != nullptr && bytes != nullptr, "null argument");
  if (!w->tiled || m == 0) {
    *bytes = 0;
    return YSCV_HIP_OK;
  }
  // a 16-byte aligned pointer stands in for the activation: alignment is checked again at run time
  Int4Scratch L = int4_scratch_layout(w, reinterpret_cast<const void *>(uintptr_t(256)), x_dtype, m, force, ctx->num_cus);
  *bytes = L.total + L.opt_bytes;
  return YSCV_HIP_OK;
}

// Runs the int4 path: activation preparation if needed, then the skinny or the GEMM kernel.
// `ws` may be null: scratch then comes from the stream-ordered allocator, so concurrent callers
// on different streams never share it.
int32_t int4_run_ws(const yscv_hip_int4_weight *w, const void *x, int x_dtype, void *y, int y_dtype, size_t m,
                    int force /*0 auto, 1 skinny, 2 gemm*/, int epi, void *ws, size_t ws_bytes, hipStream_t s,
                    const NormFold *nf) {
  const Context *ctx = nullptr;
  YSCV_TRY(ensure_context(&ctx));
  YSCV_REQUIRE(w != nullptr, "null int4 weight handle");
  YSCV_REQUIRE(x != nullptr && y != nullptr, "null activation / output pointer");
  YSCV_REQUIRE(valid_act_dtype(x_dtype) && valid_act_dtype(y_dtype), "unknown dtype code");
  if (m == 0) return YSCV_HIP_OK;
  if (force == 1 && m > 16) return set_error(YSCV_HIP_ERR_INVALID_ARG, "gemv entry point handles m <= 16, got %zu", m);
  if (nf && (!w->tiled || m > 16 || x_dtype != YSCV_HIP_F16))
    return set_error(YSCV_HIP_ERR_UNSUPPORTED, "the folded norm exists for the skinny kernel on fp16 activations only");
  if (!w->tiled) {
    if (epi != EPI_STORE) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "fused epilogues need the tiled layout");
    note_int4_fallback();
    return launch_int4_generic(w, x, x_dtype, y, y_dtype, m, s);
  }
  note_int4_fast();
  Int4Scratch L = int4_scratch_layout(w, x, x_dtype, m, force, ctx->num_cus);
  // above 16 rows the LDS-ring GEMM (16-bit activations) has the add and SwiGLU epilogues; the exact-scale kernel has none
  if (!L.skinny && epi != EPI_STORE && !(x_dtype != YSCV_HIP_F32 && nf == nullptr))
    return set_error(YSCV_HIP_ERR_UNSUPPORTED, "fused epilogues above 16 rows need 16-bit activations");
  // f32 activations that stay on the exact-scale route (f32 scales, or an output the ring GEMM cannot take): up to
  // 128 rows go through the skinny kernel 16 rows at a time.  Each pass streams the weights again, which is still
  // 5-10 x faster than the exact-scale GEMM kernel there: that one keeps a 64 x 256 tile per workgroup and cannot fill
  // the GPU with so few rows (m = 64 against 14336 x 4096: 432 us; four skinny passes: about 60 us).
  if (!L.skinny && force == 0 && x_dtype == YSCV_HIP_F32 && m <= kChunkedSkinnyMaxRows) {
    const bool ring_ok = w->scale_dtype == YSCV_HIP_F16 &&
                         int4_gemm_ring_eligible(w, reinterpret_cast<const _Float16 *>(uintptr_t(256)), y, y_dtype, 1, m, L.k_pad);
    if (!ring_ok) {
      const size_t ysz = dtype_size(y_dtype);
      for (size_t r0 = 0; r0 < m; r0 += 16) {
        const size_t rows = m - r0 < 16 ? m - r0 : 16;
        YSCV_TRY(int4_run_ws(w, static_cast<const char *>(x) + r0 * w->k * sizeof(float), x_dtype,
                             static_cast<char *>(y) + r0 * w->n * ysz, y_dtype, rows, 1, epi, ws, ws_bytes, s));
      }
      return YSCV_HIP_OK;
    }
  }
  char *scratch = static_cast<char *>(ws);
  bool own = false;
  size_t have = ws_bytes;
  if (L.total + L.opt_bytes > 0) {
    if (scratch) {
      YSCV_REQUIRE(ws_bytes >= L.total + L.opt_bytes, "workspace too small: %zu < %zu bytes", ws_bytes, L.total + L.opt_bytes);
      YSCV_REQUIRE((reinterpret_cast<uintptr_t>(scratch) & 255) == 0, "workspace must be 256-byte aligned");
    } else {
      have = L.total + L.opt_bytes;
      YSCV_HIP_TRY(hipMallocAsync(reinterpret_cast<void **>(&scratch), have, s));
      own = true;
    }
  }
  // the GEMM's K-split partials sit behind everything else
  float *gemm_partial = (scratch != nullptr && L.opt_bytes > 0 && have >= L.total + L.opt_bytes)
                            ? reinterpret_cast<float *>(scratch + L.total) : nullptr;
  const void *xraw = (L.direct && x_dtype != YSCV_HIP_F16) ? x : nullptr;
  const _Float16 *xh = L.direct ? static_cast<const _Float16 *>(x) : reinterpret_cast<_Float16 *>(scratch);
  _Float16 *xl = (!L.direct && L.split == 2) ? reinterpret_cast<_Float16 *>(scratch + L.xh_bytes) : nullptr;
  float *row_scale = L.direct ? nullptr : reinterpret_cast<float *>(scratch + L.xh_bytes * L.split);
  float *partial = L.part_bytes ? reinterpret_cast<float *>(scratch + L.xh_bytes * L.split + L.rs_bytes) : nullptr;
  // f32 activations with more than 16 rows against a weight whose scales are stored as fp16 (the MatMulNBits form) go
  // to the LDS-ring GEMM as ONE fp16 operand: that kernel folds the group scale into fp16 weights (2^-11 relative per
  // weight), which a lo half of the activations could not refine, and it is 3.5x (prefill shapes) to 14x (few rows,
  // wide N) faster than the exact-scale kernel.  Weights with f32 scales -- what packed_int4_gemm_dispatch hands
  // over -- keep the exact-scale kernel with hi + lo activations: the reference's own test holds that entry point
  // to 1e-3 absolute (int4_matmul.rs:816-855).  The scratch keeps the size of the two-operand form.
  int run_split = L.split;
  if (!L.skinny && x_dtype == YSCV_HIP_F32 && m > 16 && w->scale_dtype == YSCV_HIP_F16 &&
      int4_gemm_ring_eligible(w, xh, y, y_dtype, 1, m, L.k_pad)) {
    run_split = 1;
    xl = nullptr;
  }
  int32_t st = YSCV_HIP_OK;
  if (!L.direct)
    st = launch_x_prep(x, x_dtype, m, w->k, L.k_pad, run_split, const_cast<_Float16 *>(xh), xl, row_scale, s);
  if (st == YSCV_HIP_OK) {
    if (L.skinny)
      st = launch_int4_skinny(w, L.plan, xh, xl, xraw, row_scale, L.k_pad, L.split, y, y_dtype, m, partial, epi, s, nf);
    else
      st = launch_int4_gemm(w, xh, xl, row_scale, L.k_pad, run_split, y, y_dtype, m, s, epi, gemm_partial, L.opt_bytes);
  }
  if (own) {
    hipError_t fe = hipFreeAsync(scratch, s);
    YSCV_TRY(st);
    YSCV_HIP_TRY(fe);
  }
  return st;
}

static int32_t int4_run(const yscv_hip_int4_weight *w, const void *x, int x_dtype, void *y, int y_dtype,
                        size_t m, int force, hipStream_t s) {
  return int4_run_ws(w, x, x_dtype, y, y_dtype, m, force, EPI_STORE, nullptr, 0, s);
}

static void free_int4(yscv_hip_int4_weight *w) {
  if (!w) return;
  (void)hipFree(w->tiles);
  (void)hipFree(w->tscales);
  (void)hipFree(w->tzps);
  (void)hipFree(w->raw);
  (void)hipFree(w->rscales);
  (void)hipFree(w->rzps);
  delete w;
}

static int32_t int4_create(const uint8_t *packed, const void *scales, int32_t scale_dtype,
                           const uint8_t *zero_points, int32_t nibble_format, size_t n, size_t k,
                           size_t g, yscv_hip_int4_weight **out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(out != nullptr, "null output handle pointer");
  *out = nullptr;
  YSCV_REQUIRE(packed && scales, "null packed / scales pointer");
  YSCV_REQUIRE(n > 0 && k > 0, "empty weight (n=%zu k=%zu)", n, k);
  YSCV_REQUIRE(g > 0 && g % 2 == 0, "group_size must be even and > 0, got %zu", g);
  YSCV_REQUIRE(k % g == 0, "group_size %zu does not divide k %zu", g, k);
  YSCV_REQUIRE(scale_dtype == YSCV_HIP_F32 || scale_dtype == YSCV_HIP_F16, "scales must be f32 or f16");
  YSCV_REQUIRE(nibble_format == YSCV_HIP_NIBBLE_SIGNED || nibble_format == YSCV_HIP_NIBBLE_UNSIGNED,
               "unknown nibble format %d", nibble_format);
  YSCV_REQUIRE(!(zero_points && nibble_format == YSCV_HIP_NIBBLE_SIGNED),
               "zero points are only defined for unsigned nibbles");
  YSCV_REQUIRE(n < (1u << 30) && k < (1u << 30), "dimension too large");
  const size_t groups = k / g;
  const size_t zp_row = (groups + 1) / 2;
  bool has_zp = false;
  if (zero_points) {
    for (size_t row = 0; row < n && !has_zp; row++)
      for (size_t grp = 0; grp < groups; grp++) {
        uint8_t b = zero_points[row * zp_row + grp / 2];
        if (((grp & 1) ? (b >> 4) : (b & 15)) != 8) {
          has_zp = true;
          break;
        }
      }
  }
  auto *w = new yscv_hip_int4_weight();
  w->n = n;
  w->k = k;
  w->g = g;
  w->scale_dtype = scale_dtype;
  w->has_zp = has_zp;
  w->tiled = (g == 32 || g == 64 || g % 128 == 0);
  const size_t ssz = dtype_size(scale_dtype);
  hipStream_t s = nullptr;

  DevBuf d_packed, d_scales, d_zp_packed, d_zp;
  int32_t st = d_packed.alloc(n * k / 2);
  if (st == YSCV_HIP_OK) st = d_scales.alloc(n * groups * ssz);
  if (st != YSCV_HIP_OK) {
    free_int4(w);
    return st;
  }
#define CREATE_TRY(expr)                                                                       \
  do {                                                                                         \
    hipError_t _e = (expr);                                                                    \
    if (_e != hipSuccess) {                                                                    \
      free_int4(w);                                                                            \
      return set_error(_e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE,     \
                       "%s failed: %s", #expr, hipGetErrorString(_e));                         \
    }                                                                                          \
  } while (0)
#define CREATE_ST(expr)            \
  do {                             \
    int32_t _s = (expr);           \
    if (_s != YSCV_HIP_OK) {       \
      free_int4(w);                \
      return _s;                   \
    }                              \
  } while (0)
  CREATE_TRY(hipMemcpy(d_packed.p, packed, n * k / 2, hipMemcpyHostToDevice));
  CREATE_TRY(hipMemcpy(d_scales.p, scales, n * groups * ssz, hipMemcpyHostToDevice));
  if (has_zp) {
    CREATE_ST(d_zp_packed.alloc(n * zp_row));
    CREATE_ST(d_zp.alloc(n * groups));
    CREATE_TRY(hipMemcpy(d_zp_packed.p, zero_points, n * zp_row, hipMemcpyHostToDevice));
    CREATE_ST(launch_unpack_zps(d_zp_packed.as<uint8_t>(), n, groups, d_zp.as<uint8_t>(), s));
  }
  if (w->tiled) {
    w->gm = g == 32 ? GM32 : (g == 64 ? GM64 : GM128);
    w->nt = ceil_div(n, (size_t)16);
    w->kt = ceil_div(k, (size_t)128);
    w->ktp = round_up(w->kt, (size_t)4);
    w->chunks = w->gm == GM128 ? ceil_div(w->ktp, g / 128) : w->ktp;
    const int spt = scales_per_chunk(w->gm);
    const size_t tile_bytes = w->nt * w->ktp * (size_t)kTileBytes;
    const size_t sc_elems = w->nt * w->chunks * 16 * (size_t)spt;
    CREATE_TRY(hipMalloc(reinterpret_cast<void **>(&w->tiles), tile_bytes));
    CREATE_TRY(hipMalloc(&w->tscales, sc_elems * ssz));
    if (has_zp) CREATE_TRY(hipMalloc(reinterpret_cast<void **>(&w->tzps), sc_elems));
    CREATE_ST(launch_int4_retile(d_packed.as<uint8_t>(), nibble_format, n, k, w->nt, w->ktp, w->tiles, s));
    CREATE_ST(launch_int4_retile_scales(d_scales.p, scale_dtype, has_zp ? d_zp.as<uint8_t>() : nullptr, n, k, g,
                                        w->gm, w->nt, w->chunks, w->tscales, w->tzps, s));
    w->device_bytes = tile_bytes + sc_elems * ssz + (has_zp ? sc_elems : 0);
  } else {
    // generic layout: keep the uploaded buffers themselves
    if (nibble_format == YSCV_HIP_NIBBLE_SIGNED) CREATE_ST(launch_xor88(d_packed.as<uint8_t>(), n * k / 2, s));
    w->raw = d_packed.as<uint8_t>();
    d_packed.p = nullptr;
    w->rscales = d_scales.p;
    d_scales.p = nullptr;
    if (has_zp) {
      w->rzps = d_zp.as<uint8_t>();
      d_zp.p = nullptr;
    }
    w->device_bytes = n * k / 2 + n * groups * ssz + (has_zp ? n * groups : 0);
  }
  CREATE_TRY(hipStreamSynchronize(s));
#undef CREATE_TRY
#undef CREATE_ST
  *out = w;
  return YSCV_HIP_OK;
}

// Tiled weight from buffers that are already on the device (unsigned or signed nibbles in natural
// [n][k/2] order, scales [n][k/g]); no zero points.  Used by the decoder's on-device random initialisation.
int32_t int4_create_from_device(const uint8_t *d_packed, const void *d_scales, int scale_dtype, int nibble_format,
                                size_t n, size_t k, size_t g, yscv_hip_int4_weight **out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(out && d_packed && d_scales, "null argument");
  *out = nullptr;
  YSCV_REQUIRE(g == 32 || g == 64 || g % 128 == 0, "device-side creation needs a tiled group size");
  YSCV_REQUIRE(k % g == 0 && n > 0 && k > 0, "bad shape n=%zu k=%zu group=%zu", n, k, g);
  auto *w = new yscv_hip_int4_weight();
  w->n = n;
  w->k = k;
  w->g = g;
  w->scale_dtype = scale_dtype;
  w->has_zp = false;
  w->tiled = true;
  w->gm = g == 32 ? GM32 : (g == 64 ? GM64 : GM128);
  w->nt = ceil_div(n, (size_t)16);
  w->kt = ceil_div(k, (size_t)128);
  w->ktp = round_up(w->kt, (size_t)4);
  w->chunks = w->gm == GM128 ? ceil_div(w->ktp, g / 128) : w->ktp;
  const size_t ssz = dtype_size(scale_dtype);
  const size_t tile_bytes = w->nt * w->ktp * (size_t)kTileBytes;
  const size_t sc_elems = w->nt * w->chunks * 16 * (size_t)scales_per_chunk(w->gm);
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&w->tiles), tile_bytes);
  if (e == hipSuccess) e = hipMalloc(&w->tscales, sc_elems * ssz);
  if (e != hipSuccess) {
    free_int4(w);
    return set_error(e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE, "weight allocation failed: %s",
                     hipGetErrorString(e));
  }
  int32_t st = launch_int4_retile(d_packed, nibble_format, n, k, w->nt, w->ktp, w->tiles, nullptr);
  if (st == YSCV_HIP_OK)
    st = launch_int4_retile_scales(d_scales, scale_dtype, nullptr, n, k, g, w->gm, w->nt, w->chunks, w->tscales, nullptr, nullptr);
  if (st != YSCV_HIP_OK) {
    free_int4(w);
    return st;
  }
  w->device_bytes = tile_bytes + sc_elems * ssz;
  *out = w;
  return YSCV_HIP_OK;
}

static void free_i8(yscv_hip_i8_weight *b) {
  if (!b) return;
  (void)hipFree(b->frag);
  (void)hipFree(b->col_sum);
  delete b;
}

}  // namespace yscv

using namespace yscv;

extern "C" {

// ---- lifecycle ---------------------------------------------------------------------------
int32_t yscv_hip_init(int32_t device_index) { return init_context(device_index); }

int32_t yscv_hip_shutdown(void) {
  drop_context();
  return YSCV_HIP_OK;
}

uint32_t yscv_hip_abi_version(void) { return YSCV_HIP_ABI_VERSION; }

const char *yscv_hip_last_error(void) { return last_error_slot().c_str(); }

int32_t yscv_hip_device_info(char *buf, size_t buf_len) {
  const Context *ctx = nullptr;
  YSCV_TRY(ensure_context(&ctx));
  YSCV_REQUIRE(buf && buf_len > 0, "null buffer");
  snprintf(buf, buf_len,
           "device=%d name=\"%s\" arch=%s compute_units=%d lds_per_block=%d hbm_bytes=%zu "
           "int4_skinny=mfma_f32_16x16x32_f16 int4_gemm=mfma_f32_16x16x32_f16 int8_gemm=mfma_i32_16x16x64_i8",
           ctx->device, ctx->name, ctx->arch, ctx->num_cus, ctx->lds_bytes, ctx->total_mem);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_malloc(void **dev_ptr, size_t bytes) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(dev_ptr != nullptr, "null pointer");
  YSCV_HIP_TRY(hipMalloc(dev_ptr, bytes ? bytes : 4));
  return YSCV_HIP_OK;
}
int32_t yscv_hip_free(void *dev_ptr) {
  YSCV_HIP_TRY(hipFree(dev_ptr));
  return YSCV_HIP_OK;
}
int32_t yscv_hip_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, as_stream(stream)));
  YSCV_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
  return YSCV_HIP_OK;
}
int32_t yscv_hip_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
  YSCV_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
  return YSCV_HIP_OK;
}
int32_t yscv_hip_stream_synchronize(void *stream) {
  YSCV_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
  return YSCV_HIP_OK;
}

// ---- int4 ------------------------------------------------------------------------------------
int32_t yscv_hip_int4_weight_create(const uint8_t *packed, const void *scales, int32_t scale_dtype,
                                    const uint8_t *zero_points, int32_t nibble_format, size_t n, size_t k,
                                    size_t group_size, yscv_hip_int4_weight **out) {
  return int4_create(packed, scales, scale_dtype, zero_points, nibble_format, n, k, group_size, out);
}

int32_t yscv_hip_int4_weight_destroy(yscv_hip_int4_weight *w) {
  free_int4(w);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_int4_weight_dims(const yscv_hip_int4_weight *w, size_t *n, size_t *k, size_t *group_size,
                                  size_t *device_bytes) {
  YSCV_REQUIRE(w != nullptr, "null int4 weight handle");
  if (n) *n = w->n;
  if (k) *k = w->k;
  if (group_size) *group_size = w->g;
  if (device_bytes) *device_bytes = w->device_bytes;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_int4_matmul(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype, void *y_dev,
                             int32_t y_dtype, size_t m, void *stream) {
  return int4_run(w, x_dev, x_dtype, y_dev, y_dtype, m, 0, as_stream(stream));
}
int32_t yscv_hip_int4_gemv(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype, void *y_dev,
                           int32_t y_dtype, size_t m, void *stream) {
  return int4_run(w, x_dev, x_dtype, y_dev, y_dtype, m, 1, as_stream(stream));
}
int32_t yscv_hip_int4_gemm(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype, void *y_dev,
                           int32_t y_dtype, size_t m, void *stream) {
  return int4_run(w, x_dev, x_dtype, y_dev, y_dtype, m, 2, as_stream(stream));
}

int32_t yscv_hip_int4_matmul_fused(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype, void *y_dev,
                                   int32_t y_dtype, size_t m, int32_t epilogue, void *stream) {
  YSCV_REQUIRE(epilogue == YSCV_HIP_EPILOGUE_STORE || epilogue == YSCV_HIP_EPILOGUE_ADD_F32 ||
                   epilogue == YSCV_HIP_EPILOGUE_SWIGLU,
               "unknown epilogue %d", epilogue);
  YSCV_REQUIRE(m <= 16 || x_dtype != YSCV_HIP_F32 || epilogue == YSCV_HIP_EPILOGUE_STORE,
               "fused epilogues with f32 activations run on the skinny kernel: m <= 16, got %zu", m);
  return int4_run_ws(w, x_dev, x_dtype, y_dev, y_dtype, m, m <= 16 ? 1 : 0, epilogue, nullptr, 0, as_stream(stream));
}

int32_t yscv_hip_int4_matmul_static(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype, void *y_dev,
                                    int32_t y_dtype, size_t m, void *stream) {
  const Context *ctx = nullptr;
  YSCV_TRY(ensure_context(&ctx));
  YSCV_REQUIRE(w != nullptr && x_dev != nullptr && y_dev != nullptr, "null argument");
  YSCV_REQUIRE(valid_act_dtype(x_dtype) && valid_act_dtype(y_dtype), "unknown dtype code");
  if (m == 0) return YSCV_HIP_OK;
  void *ws = ctx->device < kMaxDevices ? g_scratch_ptr[ctx->device] : nullptr;
  if (ws == nullptr) return set_error(YSCV_HIP_ERR_DEVICE, "the static scratch of device %d was never resolved", ctx->device);
  if (w->tiled) {
    const Int4Scratch L = int4_scratch_layout(w, x_dev, x_dtype, m, 0, ctx->num_cus);
    if (L.total + L.opt_bytes > (size_t)YSCV_HIP_STATIC_SCRATCH_BYTES)
      return set_error(YSCV_HIP_ERR_INVALID_ARG,
                       "this call needs %zu bytes of scratch, the static scratch holds %zu: use yscv_hip_int4_matmul_ws",
                       L.total + L.opt_bytes, (size_t)YSCV_HIP_STATIC_SCRATCH_BYTES);
  }
  return int4_run_ws(w, x_dev, x_dtype, y_dev, y_dtype, m, 0, EPI_STORE, ws, YSCV_HIP_STATIC_SCRATCH_BYTES, as_stream(stream));
}

int32_t yscv_hip_int4_workspace_bytes(const yscv_hip_int4_weight *w, size_t m, int32_t x_dtype, size_t *bytes) {
  return int4_workspace_bytes(w, m, x_dtype, 0, bytes);
}

int32_t yscv_hip_int4_matmul_ws(const yscv_hip_int4_weight *w, const void *x_dev, int32_t x_dtype, void *y_dev,
                                int32_t y_dtype, size_t m, void *workspace_dev, size_t workspace_bytes, void *stream) {
  YSCV_REQUIRE(workspace_dev != nullptr || workspace_bytes == 0, "null workspace with non-zero size");
  size_t need = 0;
  YSCV_TRY(int4_workspace_bytes(w, m, x_dtype, 0, &need));
  if (need > 0) YSCV_REQUIRE(workspace_dev != nullptr, "this call needs %zu bytes of workspace", need);
  return int4_run_ws(w, x_dev, x_dtype, y_dev, y_dtype, m, 0, EPI_STORE, workspace_dev, workspace_bytes,
                     as_stream(stream));
}

static int32_t int4_host_call(const uint8_t *weight_packed, const float *scales, const float *activation,
                              float *output, size_t m, size_t n, size_t k, size_t g, int force) {
  YSCV_REQUIRE(weight_packed && scales && activation && output, "null slice");
  yscv_hip_int4_weight *w = nullptr;
  YSCV_TRY(int4_create(weight_packed, scales, YSCV_HIP_F32, nullptr, YSCV_HIP_NIBBLE_SIGNED, n, k, g, &w));
  DevBuf dx, dy;
  int32_t st = dx.alloc(m * k * sizeof(float));
  if (st == YSCV_HIP_OK) st = dy.alloc(m * n * sizeof(float));
  if (st == YSCV_HIP_OK) {
    hipError_t e = hipMemcpy(dx.p, activation, m * k * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) st = set_error(YSCV_HIP_ERR_DEVICE, "H2D copy failed: %s", hipGetErrorString(e));
  }
  if (st == YSCV_HIP_OK) st = int4_run(w, dx.p, YSCV_HIP_F32, dy.p, YSCV_HIP_F32, m, force, nullptr);
  if (st == YSCV_HIP_OK) {
    hipError_t e = hipMemcpy(output, dy.p, m * n * sizeof(float), hipMemcpyDeviceToHost);
    if (e != hipSuccess) st = set_error(YSCV_HIP_ERR_DEVICE, "D2H copy failed: %s", hipGetErrorString(e));
  }
  free_int4(w);
  return st;
}

int32_t yscv_hip_packed_int4_gemv_dispatch(const uint8_t *weight_packed, const float *scales,
                                           const float *activation, float *output, size_t m_w, size_t k,
                                           size_t group_size) {
  return int4_host_call(weight_packed, scales, activation, output, 1, m_w, k, group_size, 1);
}

int32_t yscv_hip_packed_int4_gemm_dispatch(const uint8_t *weight_packed, const float *scales,
                                           const float *activation, float *output, size_t m, size_t n, size_t k,
                                           size_t group_size) {
  if (m == 0) return YSCV_HIP_OK;
  return int4_host_call(weight_packed, scales, activation, output, m, n, k, group_size, 2);
}

int32_t yscv_hip_pack_int4_symmetric_per_group(const float *weights, size_t m_w, size_t k, size_t group_size,
                                               uint8_t *packed_out, float *scales_out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(weights && packed_out && scales_out, "null slice");
  YSCV_REQUIRE(group_size > 0 && group_size % 2 == 0 && k % group_size == 0 && m_w > 0 && k > 0,
               "bad shape m_w=%zu k=%zu group=%zu", m_w, k, group_size);
  DevBuf dw, dp, ds;
  YSCV_TRY(dw.alloc(m_w * k * sizeof(float)));
  YSCV_TRY(dp.alloc(m_w * k / 2));
  YSCV_TRY(ds.alloc(m_w * (k / group_size) * sizeof(float)));
  YSCV_HIP_TRY(hipMemcpy(dw.p, weights, m_w * k * sizeof(float), hipMemcpyHostToDevice));
  YSCV_TRY(launch_pack_int4_symmetric(dw.as<float>(), m_w, k, group_size, dp.as<uint8_t>(), ds.as<float>(), nullptr));
  YSCV_HIP_TRY(hipMemcpy(packed_out, dp.p, m_w * k / 2, hipMemcpyDeviceToHost));
  YSCV_HIP_TRY(hipMemcpy(scales_out, ds.p, m_w * (k / group_size) * sizeof(float), hipMemcpyDeviceToHost));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_quantize_f32_to_int4_dev(const float *data_dev, size_t len, float scale, int8_t zero_point,
                                          uint8_t *out_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(len == 0 || (data_dev && out_dev), "null argument");
  return launch_quantize_f32_to_int4(data_dev, len, scale, (int)zero_point, out_dev, as_stream(stream));
}

int32_t yscv_hip_quantize_f32_to_int4(const float *data, size_t len, float scale, int8_t zero_point, uint8_t *output) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(len == 0 || (data && output), "null argument");
  if (len == 0) return YSCV_HIP_OK;
  DevBuf dx, dq;
  YSCV_TRY(dx.alloc(len * sizeof(float)));
  YSCV_TRY(dq.alloc((len + 1) / 2));
  YSCV_HIP_TRY(hipMemcpy(dx.p, data, len * sizeof(float), hipMemcpyHostToDevice));
  YSCV_TRY(launch_quantize_f32_to_int4(dx.as<float>(), len, scale, (int)zero_point, dq.as<uint8_t>(), nullptr));
  YSCV_HIP_TRY(hipMemcpy(output, dq.p, (len + 1) / 2, hipMemcpyDeviceToHost));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_dequantize_int4_to_f32(const uint8_t *packed, size_t n_bytes, float scale, int8_t zero_point,
                                        float *output) {
  YSCV_TRY(ensure_context(nullptr));
  if (n_bytes == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(packed && output, "null slice");
  DevBuf dp, dout;
  YSCV_TRY(dp.alloc(n_bytes));
  YSCV_TRY(dout.alloc(n_bytes * 2 * sizeof(float)));
  YSCV_HIP_TRY(hipMemcpy(dp.p, packed, n_bytes, hipMemcpyHostToDevice));
  YSCV_TRY(launch_dequantize_int4(dp.as<uint8_t>(), n_bytes, scale, (int)zero_point, dout.as<float>(), nullptr));
  YSCV_HIP_TRY(hipMemcpy(output, dout.p, n_bytes * 2 * sizeof(float), hipMemcpyDeviceToHost));
  return YSCV_HIP_OK;
}

// ---- int8 ------------------------------------------------------------------------------------
int32_t yscv_hip_pack_i8_b_for_matmul(const int8_t *b_host, size_t k, size_t n, yscv_hip_i8_weight **out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(out != nullptr, "null output handle pointer");
  *out = nullptr;
  YSCV_REQUIRE(b_host != nullptr, "null b");
  YSCV_REQUIRE(k > 0 && n > 0 && k < (1u << 30) && n < (1u << 30), "bad shape k=%zu n=%zu", k, n);
  auto *b = new yscv_hip_i8_weight();
  b->k = k;
  b->n = n;
  b->kp = round_up(k, 64);
  b->np = round_up(n, 16);
  DevBuf raw;
  int32_t st = raw.alloc(k * n);
  hipError_t e = hipSuccess;
  if (st == YSCV_HIP_OK) e = hipMemcpy(raw.p, b_host, k * n, hipMemcpyHostToDevice);
  if (st == YSCV_HIP_OK && e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&b->frag), b->kp * b->np);
  if (st == YSCV_HIP_OK && e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&b->col_sum), b->np * sizeof(int32_t));
  if (st == YSCV_HIP_OK && e == hipSuccess) st = launch_i8_pack_b(raw.as<int8_t>(), k, n, b->kp, b->np, b->frag, b->col_sum, nullptr);
  if (st == YSCV_HIP_OK && e == hipSuccess) e = hipStreamSynchronize(nullptr);
  if (st != YSCV_HIP_OK || e != hipSuccess) {
    free_i8(b);
    if (st != YSCV_HIP_OK) return st;
    return set_error(e == hipErrorOutOfMemory ? YSCV_HIP_ERR_OOM : YSCV_HIP_ERR_DEVICE, "packing B failed: %s",
                     hipGetErrorString(e));
  }
  b->device_bytes = b->kp * b->np + b->np * sizeof(int32_t);
  *out = b;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_i8_weight_destroy(yscv_hip_i8_weight *b) {
  free_i8(b);
  return YSCV_HIP_OK;
}

int32_t yscv_hip_i8_weight_dims(const yscv_hip_i8_weight *b, size_t *k, size_t *n) {
  YSCV_REQUIRE(b != nullptr, "null int8 weight handle");
  if (k) *k = b->k;
  if (n) *n = b->n;
  return YSCV_HIP_OK;
}

int32_t yscv_hip_int8_matmul(const void *a_dev, int32_t a_is_u8, int32_t a_zp, const yscv_hip_i8_weight *b, size_t m,
                             int32_t *out_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(b != nullptr, "null int8 weight handle");
  if (m == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(a_dev && out_dev, "null a / out pointer");
  YSCV_REQUIRE(a_is_u8 ? (a_zp >= 0 && a_zp <= 255) : (a_zp >= -128 && a_zp <= 127), "zero point %d out of range", a_zp);
  I8Epilogue ep{};
  ep.mode = 0;
  return launch_i8_gemm(a_dev, a_is_u8, a_zp, b, m, out_dev, ep, as_stream(stream));
}

int32_t yscv_hip_int8_matmul_requant(const void *a_dev, int32_t a_is_u8, int32_t a_zp, const yscv_hip_i8_weight *b,
                                     size_t m, const int32_t *corr_dev, const float *composite_dev, float composite,
                                     float y_zp, int32_t round_mode, int32_t clamp_lo, int32_t clamp_hi, void *out_dev,
                                     void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(b != nullptr, "null int8 weight handle");
  if (m == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(a_dev && out_dev, "null a / out pointer");
  YSCV_REQUIRE(a_is_u8 ? (a_zp >= 0 && a_zp <= 255) : (a_zp >= -128 && a_zp <= 127), "zero point %d out of range", a_zp);
  YSCV_REQUIRE(round_mode == YSCV_HIP_ROUND_HALF_AWAY || round_mode == YSCV_HIP_ROUND_TIES_EVEN, "unknown rounding mode");
  YSCV_REQUIRE(clamp_lo <= clamp_hi && ((clamp_lo >= -128 && clamp_hi <= 127) || (clamp_lo >= 0 && clamp_hi <= 255)),
               "clamp range [%d,%d] does not fit one byte", clamp_lo, clamp_hi);
  I8Epilogue ep{};
  ep.mode = 1;
  ep.corr = corr_dev;
  ep.composite_v = composite_dev;
  ep.composite = composite;
  ep.y_zp = y_zp;
  ep.round_mode = round_mode;
  ep.lo = clamp_lo;
  ep.hi = clamp_hi;
  return launch_i8_gemm(a_dev, a_is_u8, a_zp, b, m, out_dev, ep, as_stream(stream));
}

int32_t yscv_hip_int8_matmul_prepacked_dispatch(const int8_t *a, const yscv_hip_i8_weight *b, size_t m, int32_t *out) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(b != nullptr, "null int8 weight handle");
  if (m == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(a && out, "null slice");
  DevBuf da, dout;
  YSCV_TRY(da.alloc(m * b->k));
  YSCV_TRY(dout.alloc(m * b->n * sizeof(int32_t)));
  YSCV_HIP_TRY(hipMemcpy(da.p, a, m * b->k, hipMemcpyHostToDevice));
  I8Epilogue ep{};
  YSCV_TRY(launch_i8_gemm(da.p, 0, 0, b, m, dout.p, ep, nullptr));
  YSCV_HIP_TRY(hipMemcpy(out, dout.p, m * b->n * sizeof(int32_t), hipMemcpyDeviceToHost));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_int8_matmul_dispatch(const int8_t *a, const int8_t *b, size_t m, size_t k, size_t n, int32_t *out) {
  if (m == 0 || n == 0) return YSCV_HIP_OK;
  yscv_hip_i8_weight *bw = nullptr;
  YSCV_TRY(yscv_hip_pack_i8_b_for_matmul(b, k, n, &bw));
  int32_t st = yscv_hip_int8_matmul_prepacked_dispatch(a, bw, m, out);
  free_i8(bw);
  return st;
}

// ---- elementwise -----------------------------------------------------------------------------------
int32_t yscv_hip_quantize_linear_f32_to_i8(const float *data_dev, size_t len, float scale, float zero_point,
                                           int8_t *out_dev, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  if (len == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(data_dev && out_dev, "null pointer");
  return launch_quantize_linear_i8(data_dev, len, scale, zero_point, out_dev, as_stream(stream));
}

int32_t yscv_hip_requant_i8_per_channel(const int32_t *acc_dev, size_t len, const int32_t *corr_dev,
                                        const float *composite_dev, float y_zp, int8_t *out_dev, size_t c,
                                        void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  if (len == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(acc_dev && corr_dev && composite_dev && out_dev, "null pointer");
  YSCV_REQUIRE(c > 0 && len % c == 0, "len %zu is not a multiple of c %zu", len, c);
  return launch_requant(acc_dev, len, c, corr_dev, composite_dev, 0.0f, y_zp, YSCV_HIP_ROUND_TIES_EVEN, -128, 127, 0,
                        out_dev, as_stream(stream));
}

int32_t yscv_hip_requant_i32_row_to_i8(const int32_t *acc_dev, size_t len, const int32_t *bias_dev, float composite,
                                       float y_zp, int32_t relu, int8_t *out_dev, size_t c, void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  if (len == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(acc_dev && out_dev, "null pointer");
  YSCV_REQUIRE(c > 0 && len % c == 0, "len %zu is not a multiple of c %zu", len, c);
  return launch_requant(acc_dev, len, c, bias_dev, nullptr, composite, y_zp, YSCV_HIP_ROUND_TIES_EVEN, -128, 127,
                        relu ? 1 : 0, out_dev, as_stream(stream));
}

int32_t yscv_hip_dynamic_quantize_linear(const float *x_dev, size_t len, uint8_t *y_dev, float *scale_zp_dev,
                                         void *stream) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(scale_zp_dev != nullptr, "null scale/zero-point pointer");
  YSCV_REQUIRE(len == 0 || (x_dev && y_dev), "null pointer");
  return launch_dynamic_quantize_linear(x_dev, len, y_dev, scale_zp_dev, as_stream(stream));
}

int32_t yscv_hip_quantize_linear_f32_to_i8_dispatch(const float *data, size_t len, float scale, float zero_point,
                                                    int8_t *output) {
  YSCV_TRY(ensure_context(nullptr));
  if (len == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(data && output, "null slice");
  DevBuf dx, dq;
  YSCV_TRY(dx.alloc(len * sizeof(float)));
  YSCV_TRY(dq.alloc(len));
  YSCV_HIP_TRY(hipMemcpy(dx.p, data, len * sizeof(float), hipMemcpyHostToDevice));
  YSCV_TRY(launch_quantize_linear_i8(dx.as<float>(), len, scale, zero_point, dq.as<int8_t>(), nullptr));
  YSCV_HIP_TRY(hipMemcpy(output, dq.p, len, hipMemcpyDeviceToHost));
  return YSCV_HIP_OK;
}

static int32_t requant_host(const int32_t *acc, size_t len, const int32_t *corr, const float *composite_v,
                            float composite, float y_zp, int relu, int8_t *out, size_t c) {
  YSCV_TRY(ensure_context(nullptr));
  if (len == 0) return YSCV_HIP_OK;
  YSCV_REQUIRE(acc && out, "null slice");
  YSCV_REQUIRE(c > 0 && len % c == 0, "len %zu is not a multiple of c %zu", len, c);
  DevBuf da, dc, dv, dq;
  YSCV_TRY(da.alloc(len * sizeof(int32_t)));
  YSCV_TRY(dq.alloc(len));
  YSCV_HIP_TRY(hipMemcpy(da.p, acc, len * sizeof(int32_t), hipMemcpyHostToDevice));
  if (corr) {
    YSCV_TRY(dc.alloc(c * sizeof(int32_t)));
    YSCV_HIP_TRY(hipMemcpy(dc.p, corr, c * sizeof(int32_t), hipMemcpyHostToDevice));
  }
  if (composite_v) {
    YSCV_TRY(dv.alloc(c * sizeof(float)));
    YSCV_HIP_TRY(hipMemcpy(dv.p, composite_v, c * sizeof(float), hipMemcpyHostToDevice));
  }
  YSCV_TRY(launch_requant(da.as<int32_t>(), len, c, corr ? dc.as<int32_t>() : nullptr,
                          composite_v ? dv.as<float>() : nullptr, composite, y_zp, YSCV_HIP_ROUND_TIES_EVEN, -128, 127,
                          relu, dq.p, nullptr));
  YSCV_HIP_TRY(hipMemcpy(out, dq.p, len, hipMemcpyDeviceToHost));
  return YSCV_HIP_OK;
}

int32_t yscv_hip_requant_i8_per_channel_dispatch(const int32_t *acc, size_t len, const int32_t *corr,
                                                 const float *composite, float y_zp, int8_t *out, size_t c) {
  YSCV_REQUIRE(corr && composite, "null slice");
  return requant_host(acc, len, corr, composite, 0.0f, y_zp, 0, out, c);
}

int32_t yscv_hip_requant_i32_row_to_i8_dispatch(const int32_t *acc, size_t len, const int32_t *bias, float composite,
                                                float y_zp, int32_t relu, int8_t *out, size_t c) {
  return requant_host(acc, len, bias, nullptr, composite, y_zp, relu ? 1 : 0, out, c);
}

int32_t yscv_hip_dynamic_quantize_linear_host(const float *x, size_t len, uint8_t *y, float *scale, float *zero_point) {
  YSCV_TRY(ensure_context(nullptr));
  YSCV_REQUIRE(scale && zero_point, "null scale / zero-point pointer");
  YSCV_REQUIRE(len == 0 || (x && y), "null slice");
  DevBuf dx, dy, dsz;
  YSCV_TRY(dx.alloc(len * sizeof(float)));
  YSCV_TRY(dy.alloc(len));
  YSCV_TRY(dsz.alloc(2 * sizeof(float)));
  if (len) YSCV_HIP_TRY(hipMemcpy(dx.p, x, len * sizeof(float), hipMemcpyHostToDevice));
  YSCV_TRY(launch_dynamic_quantize_linear(dx.as<float>(), len, dy.as<uint8_t>(), dsz.as<float>(), nullptr));
  float sz[2];
  YSCV_HIP_TRY(hipMemcpy(sz, dsz.p, sizeof(sz), hipMemcpyDeviceToHost));
  if (len) YSCV_HIP_TRY(hipMemcpy(y, dy.p, len, hipMemcpyDeviceToHost));
  *scale = sz[0];
  *zero_point = sz[1];
  return YSCV_HIP_OK;
}

}  // extern "C"
