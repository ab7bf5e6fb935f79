// Part of gemm_bf16.hip (included there, after its epilogues and launch macro; not a unit of its own):
// several of the decode products as phases of one launch.
#pragma once

// ------------------------------------------------------------------------------ several phases, one launch

#define CHAIN_MAX_PHASES 6
#define CHAIN_SYNC_WORDS 4096          // 32-bit words the caller brings, zero before the first launch: phase p counts its
#define CHAIN_FLAGS_AT 2048            // workgroups in at word 64 p and raises its flag at word 2048 + 64 p
#define CHAIN_LDS_BYTES (160 * 1024 - 256)

struct ChainPhase {
  int kind, first, gx, waves;          // which kernel's statements, the phase's first block, its workgroups and their waves
  MidCall mid;
  RowsCall rows;
};
struct ChainArgs {
  int n, spin_limit;
  int* sync;
  int* err;
  ChainPhase ph[CHAIN_MAX_PHASES];
};

// Workgroups in block order, phase after phase.  A workgroup runs its phase's statements (waves the phase has no use
// for end at once), then counts itself in: every wave waits until its own device-scope stores are acknowledged, a
// barrier, and the first thread adds one to the phase's counter.  The last one to arrive puts the counter back to
// zero, takes down the flag its own phase waited for (every workgroup of the phase is past that wait) and raises the
// flag the next phase waits for: after the launch every word is zero again.
// (The statements are for the device pass only: they name types that the host pass does not know, and unlike those of
// the other kernels they do not all hang on a template parameter.  CH is true.)
template <bool CH>
__global__ __launch_bounds__(512) void gemm_bf16_chain_kernel(const ChainArgs c) {
#if defined(__HIP_DEVICE_COMPILE__)
  int p = 0;
#pragma unroll
  for (int i = 1; i < CHAIN_MAX_PHASES; ++i)
    if (i < c.n && (int)blockIdx.x >= c.ph[i].first) p = i;
  const ChainPhase& P = c.ph[p];
  if (wave_index() >= P.waves) return;
  const ChainCtx cc{(int)blockIdx.x - P.first, 0, 0, P.gx, 1, 1, P.waves, p > 0 ? c.sync + CHAIN_FLAGS_AT + 64 * (p - 1) : nullptr,
                    c.err, p, c.spin_limit};
  const MidCall& m = P.mid;
  const RowsCall& r = P.rows;
  switch (P.kind) {
    case CK_QKV_NARROW:
      mid_body<EPI_QKV_ROPE, 1, true, true, true, CH>(nullptr, m.w, m.out, m.M, m.N, m.K, 0, m.ldo, m.na, m.rp, MidSplitArgs{}, cc);
      break;
    case CK_QKV_WIDE:
      mid_body<EPI_QKV_ROPE, 1, true, false, true, CH>(nullptr, m.w, m.out, m.M, m.N, m.K, 0, m.ldo, m.na, m.rp, MidSplitArgs{}, cc);
      break;
    case CK_GLU:
      mid_body<EPI_SWIGLU_BF16, 1, true, false, true, CH>(nullptr, m.w, m.out, m.M, m.N, m.K, 0, m.ldo, m.na, m.rp, MidSplitArgs{}, cc);
      break;
    case CK_F32:
      mid_body<EPI_F32, 1, true, false, true, CH>(nullptr, m.w, m.out, m.M, m.N, m.K, 0, m.ldo, m.na, m.rp, MidSplitArgs{}, cc);
      break;
    case CK_BURST_ADD: burst_body<EPI_ADD_F32, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, cc); break;
    case CK_STREAM_ADD_8_8: stream_body<EPI_ADD_F32, 8, 8, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, r.S, cc); break;
    case CK_STREAM_ADD_8_16: stream_body<EPI_ADD_F32, 8, 16, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, r.S, cc); break;
    case CK_STREAM_ADD_16_8: stream_body<EPI_ADD_F32, 16, 8, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, r.S, cc); break;
    case CK_STREAM_ADD_16_16: stream_body<EPI_ADD_F32, 16, 16, CH>(r.x, r.w, r.out, r.M, r.N, r.K, r.ldx, r.ldo, r.S, cc); break;
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
  __syncthreads();
  if (threadIdx.x == 0) {
    const int blocks = (p + 1 < c.n ? c.ph[p + 1].first : (int)gridDim.x) - P.first;
    int* counter = c.sync + 64 * p;
    if (__hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == blocks - 1) {
      __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (p > 0) __hip_atomic_store(c.sync + CHAIN_FLAGS_AT + 64 * (p - 1), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (p + 1 < c.n) __hip_atomic_store(c.sync + CHAIN_FLAGS_AT + 64 * p, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
#endif
}

// (host) The chain that is open in this thread, if any: what bw_chain_begin was given, and the phases that wait.
struct ChainState {
  bool open = false;
  int* sync = nullptr;
  int* err = nullptr;
  int spin_limit = 0;
  int n = 0, blocks = 0, lds = 0;
  hipStream_t stream = nullptr;
  ChainPhase ph[CHAIN_MAX_PHASES];
};
static thread_local ChainState g_chain;

static bool chain_is_open() { return g_chain.open; }

static int chain_flush(hipStream_t s) {
  ChainState& g = g_chain;
  if (g.n == 0) return 0;
  ChainArgs a;
  a.n = g.n;
  a.spin_limit = g.spin_limit;
  a.sync = g.sync;
  a.err = g.err;
  for (int i = 0; i < g.n; ++i) a.ph[i] = g.ph[i];
  for (int i = g.n; i < CHAIN_MAX_PHASES; ++i) a.ph[i] = ChainPhase{};
  static bool allowed = false;                       // more than 64 KB of dynamic LDS has to be asked for once
  if (!allowed) {
    (void)hipFuncSetAttribute((const void*)gemm_bf16_chain_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    allowed = true;
  }
  const int blocks = g.blocks, lds = g.lds;
  hipStream_t stream = g.stream;
  g.n = g.blocks = g.lds = 0;
  (void)s;                                           // (the phases were asked for on g.stream; a caller on another stream has flushed)
  hipLaunchKernelGGL(gemm_bf16_chain_kernel<true>, dim3(blocks), dim3(512), lds, stream, a);
  return BW_LAUNCH_CHECK();
}

static int chain_append(const ChainPhase& ph, int wgs, int lds_bytes, hipStream_t s) {
  ChainState& g = g_chain;
  if (lds_bytes > CHAIN_LDS_BYTES || wgs <= 0) return -2;
  if (g.n > 0 && (g.stream != s || g.n == CHAIN_MAX_PHASES)) {
    const int rc = chain_flush(g.stream);
    if (rc) return rc;
  }
  g.stream = s;
  g.ph[g.n] = ph;
  g.ph[g.n].first = g.blocks;
  g.ph[g.n].gx = wgs;
  g.blocks += wgs;
  if (lds_bytes > g.lds) g.lds = lds_bytes;
  ++g.n;
  return 0;
}

static int chain_record_mid(int kind, const MidCall& c, int wgs, int lds_bytes, hipStream_t s) {
  ChainPhase ph{};
  ph.kind = kind;
  ph.waves = 8;
  ph.mid = c;
  return chain_append(ph, wgs, lds_bytes, s);
}

static int chain_record_rows(int kind, const RowsCall& c, int wgs, int waves, int lds_bytes, hipStream_t s) {
  if ((size_t)c.M * c.ldo * 4 >= ((size_t)1 << 31)) return -2;
  ChainPhase ph{};
  ph.kind = kind;
  ph.waves = waves;
  ph.rows = c;
  return chain_append(ph, wgs, lds_bytes, s);
}

// From bw_chain_begin to bw_chain_end (in the calling thread) the products of up to 16 rows that can run as phases
// (RMSNorm + product with SwiGLU, with a 32-bit store or with rotation and cache write; residual adds of few columns)
// are not launched when they are asked for but wait, and leave as one launch when anything else is launched through this
// library, at bw_chain_flush or at the end.  sync: CHAIN_SYNC_WORDS 32-bit words, zero before the first chain (every
// launch leaves them zero; after an error word that is not zero the caller clears them).  err: a word that gets a bit
// for every phase one of whose waits gave up after spin_limit looks.  Launches that do not come through this library
// (another library's kernels on the same stream) must not be made while phases wait: they would overtake them.
extern "C" int bw_chain_sync_words() { return CHAIN_SYNC_WORDS; }

extern "C" int bw_chain_begin(void* sync, int sync_words, void* err, int spin_limit) {
  if (g_chain.open || sync == nullptr || err == nullptr || sync_words < CHAIN_SYNC_WORDS || spin_limit < 0) return -2;
  g_chain = ChainState{};
  g_chain.open = true;
  g_chain.sync = (int*)sync;
  g_chain.err = (int*)err;
  g_chain.spin_limit = spin_limit;
  return 0;
}

extern "C" int bw_chain_flush(void* stream) { return g_chain.open ? chain_flush((hipStream_t)stream) : 0; }

// (for the launches of this library's other source files)
int bw_chain_flush_open(void* stream) { return bw_chain_flush(stream); }

extern "C" int bw_chain_end(void* stream) {
  if (!g_chain.open) return -2;
  const int rc = chain_flush((hipStream_t)stream);
  g_chain.open = false;
  return rc;
}
