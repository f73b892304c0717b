// The matmul dispatch of the reference engine (zero/engine.h:936-1251: run, matmul, matmul1, gemv1_rows; the weight
// upload of zero/engine_load.h:84-196; the MoE layer of zero/engine_moe.h:8-470), re-hosted on the HIP backend.
// Same entry points, argument meaning and error behaviour; launch shapes and tuning rules are gfx950's own.
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "arcz_scratch.h"
#include "clrt_hip.h"
#include "kernels/common.h"

#define GGML_Q4_0 2u
#define GGML_IQ3_S 21u
#define GGML_Q8_0 8u
#define GGML_Q4_K 12u
#define GGML_Q5_K 13u
#define GGML_Q6_K 14u
#define GGML_IQ4_XS 23u
#define GGML_IQ4_NL 20u
#define GGML_Q3_K 11u
#define GGML_IQ3_XXS 18u
#define GGML_MXFP4 39u
#define GGML_Q2_0 42u
#define GGML_AR4_128 0x41523447u

extern "C" int arcz_repack_planes(uint32_t type, size_t rows, int K, const uint8_t* gguf, uint8_t* out);
extern "C" size_t arcz_relayout_q4_0(uint32_t type, size_t rows, int K, const uint8_t* src, uint8_t* dst);
extern "C" size_t arcz_gguf_bytes(uint32_t type, size_t rows, int K);
extern "C" void arcz_iq3s_grid(uint32_t* out);
extern "C" void arcz_iq3xxs_grid(uint32_t* out);

// (zero/engine.h:27-34) raw = the device planes of all `rows` rows (an expert tensor holds n_expert * N rows)
struct GpuWeight {
  uint32_t type = 0;
  int N = 0, K = 0;
  cl_mem raw = nullptr;
  size_t rows = 0;
  // > 0: this matrix is the output head of a model with final-logit soft-capping (the reference's lm_head_ with
  // hp.softcap, zero/engine.h:984-990): the GEMVs (1-8 tokens) write c * tanh(v / c)
  float softcap = 0.0f;
  // Q6_K planes written out from a type with one scale per 32 values, for the GEMM forms (the kernels' -DHD forms):
  // 2 = the two sub-scales of a block are equal (IQ3_S), 1 = moreover the planes hold half the values (IQ3_XXS)
  int half_d = 0;
};

inline const char* ggml_type_name(uint32_t t) {
  return t == GGML_Q8_0 ? "Q8_0" : t == GGML_Q4_K ? "Q4_K" : t == GGML_Q5_K ? "Q5_K" : t == GGML_Q6_K ? "Q6_K" : t == GGML_IQ4_XS ? "IQ4_XS"
         : t == GGML_Q4_0 ? "Q4_0" : t == GGML_IQ3_S ? "IQ3_S" : t == GGML_IQ4_NL ? "IQ4_NL" : t == GGML_MXFP4 ? "MXFP4" : t == GGML_Q3_K ? "Q3_K" : t == GGML_IQ3_XXS ? "IQ3_XXS" : "?";
}

class Engine {
 public:
  ClRt cl_;
  bool profile = false;
  std::map<std::string, double> prof_ms;
  std::map<std::string, std::vector<double>> prof_each;  // every launch's time (for the minimum and median)
  std::map<std::string, int> prof_n;
  uint64_t rd_bytes = 0;  // GGUF bytes of the weights the GEMVs read (zero/engine.h:150-151)

  // max_chunk token rows of at most max_k values each (alloc_buffers, zero/engine_alloc.h:4-41)
  Engine(int max_chunk_, int max_k_) : max_chunk(max_chunk_), max_k(max_k_) {
    arcz::soft_fail() = true;
    cl_.soft_fail = true;
    if (!cl_.init()) throw std::runtime_error(std::string("no GPU runtime: ") + arcz_last_error());
    if (max_chunk <= 0 || max_k <= 0 || max_k % 256) throw std::invalid_argument("Engine: max_k must be a positive multiple of 256");
    // (the GEMM kernels address a chunk's int8 rows and a matrix's packed rows with 32-bit byte offsets)
    if ((uint64_t)max_chunk * (uint64_t)max_k >= (1ull << 32)) throw std::invalid_argument("Engine: a chunk of max_chunk x max_k values must stay below 4 GiB");
    alloc_activations();
    // the short-chunk GEMM's workspace, sized once for the most its launch rule can ask for (below: pieces x tiles
    // within two work-groups per compute unit, tiles of at most 128 x 128 f32), so that no matmul allocates or frees
    sk_force_ = getenv("ARCZ_Q4_SPLITK") ? atoi(getenv("ARCZ_Q4_SPLITK")) : -1;
    // the expert layer's launch-rule switches, read when the engine is made (a one-token layer is 16 us: nothing of
    // the environment is looked up per call)
    moe_dec_off_ = getenv("ARCZ_MOE_DECODE") && atoi(getenv("ARCZ_MOE_DECODE")) == 0;
    moe_dec_max_ = getenv("ARCZ_MOE_DECODE_MAX") ? atoi(getenv("ARCZ_MOE_DECODE_MAX")) : 16;
    moe_tmd_ = getenv("ARCZ_MOE_TMD") ? atoi(getenv("ARCZ_MOE_TMD")) : 0;
    moe_fuse_off_ = getenv("ARCZ_MOE_FUSE") && atoi(getenv("ARCZ_MOE_FUSE")) == 0;
    moe_qfuse_off_ = getenv("ARCZ_MOE_QFUSE") && atoi(getenv("ARCZ_MOE_QFUSE")) == 0;
    moe_pre_ = getenv("ARCZ_MOE_PRE") ? atoi(getenv("ARCZ_MOE_PRE")) != 0 : true;
    q4_wm_ = getenv("ARCZ_Q4_WM") ? atoi(getenv("ARCZ_Q4_WM")) : 0;
    q4_wm_min_ = getenv("ARCZ_Q4_WM_MIN") ? atoi(getenv("ARCZ_Q4_WM_MIN")) : 2048;
    sk_ws_bytes_ = (size_t)2 * (size_t)arcz_device_cus() * 128 * 128 * 4;
    sk_ws_ = buf(sk_ws_bytes_);
    // the codebook tables the kernels take as `tabs` (the reference's tabs_, zero/engine_setup.h): IQ3_S's 512 entries
    uint32_t grid[512 + 256];  // (and IQ3_XXS's 256 behind them)
    arcz_iq3s_grid(grid);
    arcz_iq3xxs_grid(grid + 512);
    tabs_ = buf(sizeof grid, grid);
  }
  cl_mem tabs_ = nullptr;
  // IQ3_S and Q3_K in the GEMM forms (prefill chunks, expert tiles): the matrix is first written out as Q6_K planes, value for
  // value, into xw_ -- the place of the reference's decode pass in front of its GEMM (zero/engine.h:1205-1250) -- and
  // the Q6_K kernels run on that.  xw_ is sized when such a weight is uploaded (the largest one), never in a matmul.
  cl_mem xw_ = nullptr;
  size_t xw_bytes_ = 0;
  GpuWeight gemm_form(const char* name, const GpuWeight& w) {
    if (w.type != GGML_IQ3_S && w.type != GGML_Q3_K && w.type != GGML_IQ3_XXS) return w;
    const size_t need = raw_planes_bytes(QT_Q6_K, w.rows, w.K / 256);
    if (need > xw_bytes_) throw std::logic_error("gemm_form: the expansion buffer is smaller than the weight");
    cl_kernel k = kernel("decode", "", w.type == GGML_Q3_K ? "expand_q3k" : w.type == GGML_IQ3_XXS ? "expand_iq3xxs" : "expand_iq3s");
    int rows = (int)w.rows, nsb = w.K / 256;
    if (w.type == GGML_Q3_K) set_args(k, 0, w.raw, xw_, rows, nsb);
    else set_args(k, 0, w.raw, xw_, tabs_, rows, nsb);
    size_t g1 = ((size_t)rows * nsb + 15) / 16 * 256, l1 = 256;
    run(name, k, 1, &g1, &l1);
    GpuWeight x = w;
    x.type = GGML_Q6_K;
    x.half_d = w.type == GGML_IQ3_XXS ? 1 : w.type == GGML_IQ3_S ? 2 : 0;
    x.raw = xw_;
    return x;
  }
  // (zero/engine_alloc.h:10, 39, 41: twice the size with two-pass matmul inputs, the residual's half behind the first)
  void alloc_activations() {
    const size_t M = (size_t)max_chunk, f = q2mm_ ? 2 : 1;
    aq_ = buf(M * max_k * f);
    // (+ 512 bytes: the prefill GEMM's last token tile reads its scale vectors in whole 128-token rows)
    asc_ = buf(M * (max_k / 32) * 4 * f + 512);
    absum_ = buf(M * (max_k / 16) * 2 * f);
    if (!asc_rep_) asc_rep_ = buf(M * (max_k / 32) * 4 + 512);
    if (!au_) au_ = buf(M * (max_k / 32) * 8 + 1024);  // (entries of 4 bytes, or 8: the bf16 pieces)
  }
  // Per-256 activation scales (act32 = 0: the reference's choice for insensitive inputs when its act32_all is off,
  // zero/engine.h:1254): the quantizers store one scale per superblock, asc [K/256][M]; the matmul kernels here take
  // per-32 scales, so a matmul of such a chunk first writes each scale out eight times into asc_rep_ and reads that.
  cl_mem asc_rep_ = nullptr;
  // sa * S per 32-block and token of the current matmul's input (act_usum), for the Q4_K / Q5_K prefill GEMM
  cl_mem au_ = nullptr;
  // d * sc and -(dmin * mn) per 32-block and row of the current matmul's Q4_K / Q5_K matrix (q4k_wscales), written in
  // front of a GEMM of many tokens; sized when such a matrix is uploaded (the largest one), never in a matmul
  cl_mem wsv_ = nullptr;
  size_t wsv_bytes_ = 0;
  int cur_act32_ = 1;
  bool a256_ = false;  // inside a matmul on the per-32 expansion of per-256 scales
  // Two-pass matmul inputs (zero/engine.h:1034-1075 q2_init, the mode of the reference's Gemma 4 and Qwen3 models):
  // every producer also quantizes what its int8 values miss, v - q * scale, the same way, into the second half of the
  // three buffers, and every matmul runs a second time over that half, accumulating (matmul below).
  bool q2mm_ = false;
  size_t q2_aq_ = 0, q2_sc_ = 0, q2_ab_ = 0;  // bytes
  std::string q2_defs_;
  cl_mem aq2_ = nullptr, asc2_ = nullptr, absum2_ = nullptr;  // views of the second halves
  void set_two_pass(bool on) {
    if (on == q2mm_) return;
    // (checked before anything is changed: a refusal leaves the engine as it was)
    if (on && (size_t)max_chunk * max_k >= (1ull << 31))
      throw std::invalid_argument("two-pass mode: a chunk of max_chunk x max_k values must stay below 2 GiB");
    for (cl_mem m : {aq_, asc_, absum_}) not_listed(m, "set_two_pass (the activation buffers are made anew)");
    for (cl_mem* v : {&aq2_, &asc2_, &absum2_})
      if (*v) { release(*v); *v = nullptr; }
    release(aq_); release(asc_); release(absum_);
    q2mm_ = on;
    cur_T_ = cur_K_ = cur_Mp_ = 0;
    alloc_activations();
    q2_defs_.clear();
    q2_aq_ = q2_sc_ = q2_ab_ = 0;
    if (!on) return;
    const size_t M = (size_t)max_chunk;
    q2_aq_ = M * max_k;
    q2_sc_ = M * (max_k / 32) * 4;
    q2_ab_ = M * (max_k / 16) * 2;
    q2_defs_ = " -DQ2_AQ=" + std::to_string(q2_aq_) + " -DQ2_SC=" + std::to_string(q2_sc_ / 4) + " -DQ2_AB=" +
               std::to_string(q2_ab_ / 2);
    aq2_ = view(aq_, q2_aq_, q2_aq_);
    asc2_ = view(asc_, q2_sc_, q2_sc_);
    absum2_ = view(absum_, q2_ab_, q2_ab_);
  }
  cl_mem view(cl_mem parent, size_t origin, size_t size) {  // (the reference's from(), zero/engine.h:251-252)
    cl_buffer_region r{origin, size};
    cl_int err = 0;
    cl_mem m = clCreateSubBuffer(parent, CL_MEM_READ_WRITE, CL_BUFFER_CREATE_TYPE_REGION, &r, &err);
    CL_CHECK(err);
    mems_.push_back(m);
    return m;
  }
  ~Engine() {
    for (auto& kv : kernels_) clReleaseKernel(kv.second);
    for (cl_program p : progs_) clReleaseProgram(p);
    for (auto it = mems_.rbegin(); it != mems_.rend(); ++it) clReleaseMemObject(*it);  // views before parents
  }
  Engine(const Engine&) = delete;

  int max_chunk, max_k;
  cl_mem aq_ = nullptr, asc_ = nullptr, absum_ = nullptr;
  int cur_T_ = 0, cur_K_ = 0, cur_Mp_ = 0;

  cl_mem buf(size_t bytes, const void* host = nullptr) {
    cl_mem m = cl_.buffer(CL_MEM_READ_WRITE, bytes, host);
    mems_.push_back(m);
    return m;
  }
  // A recorded launch list keeps the device addresses its kernels were given, the engine's own workspaces among them:
  // a buffer that a live list names is not freed or replaced (the list would read and write freed memory).  The call
  // that wanted to throws, with the engine as it was; free the list first.
  static void not_listed(cl_mem m, const char* what) {
    if (m && arcz_mem_listed(m))
      throw std::runtime_error(std::string(what) + ": a recorded launch list names this buffer (free the list first)");
  }
  void release(cl_mem m) {
    not_listed(m, "release");
    CL_CHECK(clReleaseMemObject(m));
    auto it = std::find(mems_.begin(), mems_.end(), m);
    if (it != mems_.end()) mems_.erase(it);
  }

  // (zero/engine_setup.h:317-362) one kernel object per (source, -D string, name)
  cl_kernel kernel(const std::string& which, const std::string& defs, const std::string& name) {
    const std::string key = which + defs + "|" + name;
    auto it = kernels_.find(key);
    if (it != kernels_.end()) return it->second;
    cl_program p = cl_.build(which, defs);  // (the module's name stands where the reference passes its source text)
    progs_.push_back(p);
    cl_kernel k = cl_.kernel(p, name.c_str());
    kernels_[key] = k;
    return k;
  }
  // (zero/engine.h:936-950)
  void run(const char* name, cl_kernel k, int dims, const size_t* gws, const size_t* lws) {
    cl_event e = nullptr;
    const bool timed = profile && !noalloc_;  // (a timed launch creates its events)
    CL_CHECK(clEnqueueNDRangeKernel(cl_.queue, k, dims, nullptr, gws, lws, 0, nullptr, timed ? &e : nullptr));
    if (timed && e) events_.push_back({name, e});
  }
  void collect_profile() {
    if (!profile) return;
    clFinish(cl_.queue);
    for (auto& [n, e] : events_) {
      const double ms = ClRt::event_ms(e);
      prof_ms[n] += ms;
      prof_n[n]++;
      prof_each[n].push_back(ms);
      clReleaseEvent(e);
    }
    events_.clear();
  }

  // ---- weights (zero/engine_load.h:84-130 upload_padded, :157-196 make_weight): the GGUF rows regrouped into the
  // device planes on the host, then one upload.  rows = N for a matrix, n_expert * N for an expert tensor.
  // AR4_128 and Q2_0 tensors become Q4_0 ones with the same values (arcz_relayout_q4_0): every kernel then sees Q4_0,
  // at 144 bytes per 256 values where the file has 132 and 72.  (The reference keeps both in kernels of their own,
  // zero/kernels/decode.cl PER32; the values and the arithmetic on them are the same.)
  static bool as_q4_0(uint32_t& type, const uint8_t*& data, size_t& nbytes, size_t rows, int K, std::vector<uint8_t>& hold) {
    if (type != GGML_AR4_128 && type != GGML_Q2_0) return false;
    const size_t want = arcz_relayout_q4_0(type, rows, K, nullptr, nullptr);
    if (!want) throw std::runtime_error("make_weight: K = " + std::to_string(K) + " is not whole blocks of this type (128 for AR4_128, 64 for Q2_0)");
    if (nbytes != want) throw std::runtime_error("make_weight: " + std::to_string(nbytes) + " bytes given, " + std::to_string(want) + " expected");
    hold.resize(rows * (size_t)(K / 32) * 18);
    arcz_relayout_q4_0(type, rows, K, data, hold.data());
    type = GGML_Q4_0;
    data = hold.data();
    nbytes = hold.size();
    return true;
  }
  GpuWeight make_weight(uint32_t type, const uint8_t* data, size_t nbytes, int N, int K, size_t rows = 0) {
    if (rows == 0) rows = (size_t)N;
    std::vector<uint8_t> as40;
    if (K > 0 && N > 0) as_q4_0(type, data, nbytes, rows, K, as40);
    if (type != GGML_Q4_0 && type != GGML_Q8_0 && type != GGML_Q4_K && type != GGML_Q5_K && type != GGML_Q6_K && type != GGML_IQ4_XS &&
        type != GGML_IQ3_S && type != GGML_IQ4_NL && type != GGML_MXFP4 && type != GGML_Q3_K && type != GGML_IQ3_XXS)
      throw std::runtime_error(std::string("unsupported weight type ") + std::to_string(type));
    // Rows of a 32-value-block type that end inside a superblock (K a multiple of 32, not of 256) are padded with zero
    // blocks to whole superblocks, as the reference's loader pads them (zero/engine_load.h:371-387 load_w_pad with
    // src/quants.h:661-671: scale bytes 0, so the added elements decode to 0): the weight then has K rounded up, and
    // the activations it meets are rows of that length whose tail is zero.
    std::vector<uint8_t> padded;
    const bool blk32 = type == GGML_Q8_0 || type == GGML_Q4_0 || type == GGML_IQ4_NL || type == GGML_MXFP4;
    if (blk32 && K > 0 && K % 256 && K % 32 == 0 && N > 0 && rows % (size_t)N == 0) {
      const int Kp = (K + 255) / 256 * 256;
      const size_t bb = arcz_gguf_bytes(type, 1, 256) / 8, rb = (size_t)(K / 32) * bb, prb = (size_t)(Kp / 32) * bb;
      if (nbytes != rows * rb)
        throw std::runtime_error("make_weight: " + std::to_string(nbytes) + " bytes given, " + std::to_string(rows * rb) + " expected");
      padded.assign(rows * prb, 0);
      for (size_t r = 0; r < rows; ++r) memcpy(&padded[r * prb], data + r * rb, rb);
      data = padded.data();
      nbytes = padded.size();
      K = Kp;
    }
    if (K <= 0 || K % 256 || N <= 0 || rows % (size_t)N)
      throw std::runtime_error("make_weight: K must be a multiple of 256 (of 32 for Q8_0, Q4_0, IQ4_NL and MXFP4, whose rows are padded)");
    if ((uint64_t)N * (uint64_t)(K / 256) * 256 >= (1ull << 32))
      throw std::runtime_error("make_weight: a matrix of " + std::to_string(N) + " x " + std::to_string(K) + " is too large for 32-bit row offsets");
    if (nbytes != arcz_gguf_bytes(type, rows, K))
      throw std::runtime_error("make_weight: " + std::to_string(nbytes) + " bytes given, " +
                               std::to_string(arcz_gguf_bytes(type, rows, K)) + " expected");
    if (rows * (size_t)(K / 256) >= (1ull << 31)) throw std::runtime_error("make_weight: too many superblocks for one tensor");
    GpuWeight w;
    w.type = type;
    w.N = N;
    w.K = K;
    w.rows = rows;
    const size_t pb = raw_planes_bytes((int)w.type, rows, K / 256);
    std::vector<uint8_t> planes(pb);
    if (arcz_repack_planes(type, rows, K, data, planes.data()) != 0) throw std::runtime_error("make_weight: repack failed");
    w.raw = buf(pb, planes.data());
    if ((type == GGML_Q4_K || type == GGML_Q5_K) && rows == (size_t)N) {  // (room for its rows' scale vectors, gemm_dense)
      // (with per-256 activation scales also d, an f32 per superblock and row: half a byte more per block and row)
      const size_t need = (size_t)N * (K / 32) * 21 + 4096;  // (4 + 4 bytes a block and row, or 4 + 16: the bf16 pieces)
      if (need > wsv_bytes_) {
        if (wsv_) release(wsv_);
        wsv_ = nullptr;
        wsv_bytes_ = 0;
        wsv_ = buf(need);
        wsv_bytes_ = need;
      }
    }
    if (type == GGML_IQ3_S || type == GGML_Q3_K || type == GGML_IQ3_XXS) {  // (room for its GEMM form)
      const size_t need = raw_planes_bytes(QT_Q6_K, rows, K / 256);
      if (need > xw_bytes_) {
        if (xw_) release(xw_);
        xw_ = nullptr;
        xw_bytes_ = 0;
        xw_ = buf(need);
        xw_bytes_ = need;
      }
    }
    return w;
  }
  void free_weight(GpuWeight& w) {
    if (w.raw) release(w.raw);
    w.raw = nullptr;
  }
  static uint64_t raw_bytes(const GpuWeight& w) { return arcz_gguf_bytes(w.type, w.rows, w.K); }  // (zero/engine.h:209)

  // ---- activations.  The reference quantizes inside its norm / SwiGLU kernels (quant_store16, zero/kernels/ops.cl:
  // 38-72, launched by rmsnorm_quant, zero/engine.h:1256-1267); quantize_rows is that step alone: rows [0, T) of x
  // (row stride ldx floats) into aq_ / asc_ / absum_ laid out for Mp rows, rows [T, Mp) zero.  Sets the form the next
  // matmul takes (cur_T_).
  void quantize_rows(cl_mem x, int ldx, int K, int Mp, int T, int act32) {
    check_chunk(K, Mp, T);
    if (!act32 && q2mm_) throw std::runtime_error("quantize_rows: two-pass inputs take per-32 activation scales (act32)");
    if (ldx < K || arcz_mem_size(x) < ((size_t)(T - 1) * ldx + K) * 4) throw std::runtime_error("quantize_rows: x is too small");
    cl_kernel k = kernel("ops", q2_defs_, "quant_rows");
    set_args(k, 0, x, ldx, K, Mp, T, aq_, asc_, absum_, act32);
    size_t gws[2] = {(size_t)256 * (K / 256), (size_t)(Mp + 63) / 64}, lws[2] = {256, 1};
    run("quant_rows", k, 2, gws, lws);
    cur_T_ = T; cur_K_ = K; cur_Mp_ = Mp; cur_act32_ = act32 ? 1 : 0;
  }
  // The fused producers of the reference (rmsnorm_quant, zero/engine.h:1256-1267; swiglu_quant via run_rows_quant,
  // zero/engine.h:1404-1440): a work-group per row of the chunk, or -- a pass of 1-8 tokens -- the valid rows only,
  // their superblocks over several work-groups (the GEMVs read nothing else).
  static bool wide_rows(int T) { return T <= 8; }
  // the 16-rows-a-work-group forms: one-pass engines, chunks of at least 256 rows in multiples of 16, rows of up to
  // kmax values (the kernels' R16_KMAX_NORM and R16_KMAX)
  bool rows16(int K, int Mp, int T, int kmax) const {
    static const bool off = getenv("ARCZ_PROD_R16") && atoi(getenv("ARCZ_PROD_R16")) == 0;
    return !off && !q2mm_ && !wide_rows(T) && Mp % 16 == 0 && Mp >= 256 && K <= kmax;
  }
  void rmsnorm_quant(cl_mem x, int row_off, cl_mem w, int K, int Mp, int T, int act32, float eps, cl_mem hout = nullptr) {
    check_chunk(K, Mp, T);
    if (!act32 && q2mm_) throw std::runtime_error("rmsnorm_quant: two-pass inputs take per-32 activation scales (act32)");
    if (row_off < 0 || arcz_mem_size(x) < (size_t)(row_off + T) * K * 4 || arcz_mem_size(w) < (size_t)K * 4 ||
        (hout && arcz_mem_size(hout) < (size_t)Mp * K * 4))
      throw std::runtime_error("rmsnorm_quant: a buffer is too small for " + std::to_string(T) + " rows of " + std::to_string(K));
    // (chunks: 16 rows a work-group, their scales and sums written in pieces of 16 rows; ARCZ_PROD_R16=0: a row a
    //  work-group)
    const bool r16 = rows16(K, Mp, T, 16384);
    cl_kernel k = r16 ? kernel("ops", "", "rmsnorm_quant_r16") : kernel("ops", q2_defs_, "rmsnorm_quant");
    int wh = hout ? 1 : 0;
    set_args(k, 0, x, row_off, w, K, Mp, T, eps, aq_, asc_, absum_, hout, wh, act32);
    size_t gws[2] = {256, (size_t)Mp}, lws[2] = {256, 1};
    if (r16) gws[1] = (size_t)Mp / 16;
    if (wide_rows(T)) {
      gws[0] = 256 * (size_t)((K / 256 + 15) / 16);
      gws[1] = (size_t)T;
    }
    run("rmsnorm_quant", k, 2, gws, lws);
    cur_T_ = T; cur_K_ = K; cur_Mp_ = Mp; cur_act32_ = act32 ? 1 : 0;
  }
  // gu: rows [gate(F) | up(F)] f32, or rows of F values when the matmul before has fused the product
  void swiglu_quant(cl_mem gu, int F, int Mp, int T, int act32, int fused, int gelu) {
    check_chunk(F, Mp, T);
    if (!act32 && q2mm_) throw std::runtime_error("swiglu_quant: two-pass inputs take per-32 activation scales (act32)");
    if (arcz_mem_size(gu) < (size_t)T * F * (fused ? 1 : 2) * 4) throw std::runtime_error("swiglu_quant: gu is too small");
    const bool r16 = rows16(F, Mp, T, 20480);
    cl_kernel k = r16 ? kernel("ops", "", "swiglu_quant_r16") : kernel("ops", q2_defs_, "swiglu_quant");
    set_args(k, 0, gu, F, Mp, T, aq_, asc_, absum_, act32, fused, gelu);
    size_t gws[2] = {256, (size_t)Mp}, lws[2] = {256, 1};
    if (r16) gws[1] = (size_t)Mp / 16;
    if (wide_rows(T)) {
      gws[0] = 256 * (size_t)((F / 256 + 15) / 16);
      gws[1] = (size_t)T;
    }
    run("swiglu_quant", k, 2, gws, lws);
    cur_T_ = T; cur_K_ = F; cur_Mp_ = Mp; cur_act32_ = act32 ? 1 : 0;
  }
  // x = (x + rmsnorm(t) * w) * s over the first T rows ([T][K] f32 each), then the next matmul's input from the new x:
  // rmsnorm(x) * w2, or x itself with norm2 = false (zero/engine.h:1393-1403 add_norm_quant, whose x_ and big_ are the
  // residual stream and the block's output; here they are arguments).
  void add_norm_quant(cl_mem x, cl_mem t, cl_mem w, int K, int T, int Mp, float s, cl_mem w2, bool norm2, int act32,
                      float eps) {
    check_chunk(K, Mp, T);
    if (!act32 && q2mm_) throw std::runtime_error("add_norm_quant: two-pass inputs take per-32 activation scales (act32)");
    if (arcz_mem_size(x) < (size_t)T * K * 4 || arcz_mem_size(t) < (size_t)T * K * 4 || arcz_mem_size(w) < (size_t)K * 4 ||
        (norm2 && (!w2 || arcz_mem_size(w2) < (size_t)K * 4)))
      throw std::runtime_error("add_norm_quant: a buffer is too small for " + std::to_string(T) + " rows of " + std::to_string(K));
    cl_kernel k = kernel("ops", q2_defs_, "add_norm_quant");
    int nrm = norm2 ? 1 : 0, MM = Mp, TT = T, KK = K;
    set_args(k, 0, x, t, w, KK, eps, s, w2, nrm, MM, aq_, asc_, absum_, act32, TT);
    // (a pass of 1-8 tokens: the valid rows only, as the reference; a longer chunk: all Mp rows, the padding as zeros)
    size_t gws[2] = {256, (size_t)(wide_rows(T) ? T : Mp)}, lws[2] = {256, 1};
    run("add_rmsnorm", k, 2, gws, lws);
    cur_T_ = T; cur_K_ = K; cur_Mp_ = Mp; cur_act32_ = act32 ? 1 : 0;
  }
  // Activations quantized elsewhere (the reference's benches quantize on the host, bench/gemv_bench.cpp:103-129).
  void set_activations(const int8_t* aq, const float* asc, const int16_t* absum, int K, int Mp, int T) {
    check_chunk(K, Mp, T);
    if (q2mm_) throw std::runtime_error("set_activations: a two-pass engine takes its inputs from the quantizing kernels");
    CL_CHECK(clEnqueueWriteBuffer(cl_.queue, aq_, CL_TRUE, 0, (size_t)Mp * K, aq, 0, nullptr, nullptr));
    CL_CHECK(clEnqueueWriteBuffer(cl_.queue, asc_, CL_TRUE, 0, (size_t)Mp * (K / 32) * 4, asc, 0, nullptr, nullptr));
    CL_CHECK(clEnqueueWriteBuffer(cl_.queue, absum_, CL_TRUE, 0, (size_t)Mp * (K / 16) * 2, absum, 0, nullptr, nullptr));
    cur_T_ = T; cur_K_ = K; cur_Mp_ = Mp; cur_act32_ = 1;
  }

  // ---- matmul (zero/engine.h:1080-1112): C[:, c_off : c_off+N] (+)= act * W^T for the current chunk.  acc: 0 = store,
  // 1 = accumulate into C, 2 = C = silu(C) * result (GEMM path only).  With two-pass inputs the residual's half goes
  // through the same kernels a second time and accumulates; for 1-4 tokens the GEMV takes both halves in one launch
  // (as 2 T token slots, over one read of the weights: the reference's q2_fuse_, zero/engine.h:1086-1088) whenever the
  // LDS-staged kernel can hold them, and says so in q2_fused_.  q2_nofuse_ (or ARCZ_Q2_FUSE=0): always two launches.
  bool q2_fuse_ = false, q2_fused_ = false, q2_nofuse_ = false;
  bool q2_nocap_ = false;  // (a two-pass output head: both passes run without the cap, softcap_rows caps their sum)
  // (zero/engine.h:984-990 head_defs) the GEMVs' -DSOFTCAP for an output head with a cap
  std::string head_defs(const GpuWeight& w) const {
    if (w.softcap <= 0.0f || q2_nocap_) return "";
    char b[48];
    snprintf(b, sizeof b, " -DSOFTCAP=%.9ef", w.softcap);
    return b;
  }
  void matmul(const char* name, const GpuWeight& w, int Mp, cl_mem C, int ldc, int c_off, int acc, bool act32) {
    static const bool fuse_off = getenv("ARCZ_Q2_FUSE") && atoi(getenv("ARCZ_Q2_FUSE")) == 0;
    if (q2mm_ && acc > 1) throw std::logic_error(std::string("two-pass activations with a fused epilogue: ") + name);
    if ((act32 ? 1 : 0) != cur_act32_)
      throw std::runtime_error(std::string("matmul ") + name + ": the chunk was quantized with " + (cur_act32_ ? "per-32" : "per-256") +
                               " scales, the call says " + (act32 ? "per-32" : "per-256"));
    if (!act32) {  // (one-pass engines only: the quantizers refuse it otherwise)
      cl_kernel k = kernel("ops", "", "asc_expand");
      int MM = cur_Mp_, nsb = cur_K_ / 256;
      set_args(k, 0, asc_, asc_rep_, MM, nsb);
      size_t g1 = ((size_t)nsb * 8 * MM + 255) / 256 * 256, l1 = 256;
      run("asc_expand", k, 1, &g1, &l1);
      const cl_mem s0 = asc_;
      asc_ = asc_rep_;
      a256_ = true;
      try {
        matmul1(name, w, Mp, C, ldc, c_off, acc, true);
      } catch (...) {
        asc_ = s0;
        a256_ = false;
        throw;
      }
      asc_ = s0;
      a256_ = false;
      return;
    }
    // (the output head with a logit soft cap and two-pass inputs: the cap applies to the sum of both passes, so both
    //  run without it and softcap_rows caps the sum; zero/engine.h:1081-1110)
    const bool cap = q2mm_ && w.softcap > 0.0f;
    // (only the GEMVs of 1-8 tokens cap their results -- the reference's engine never runs a head over more rows,
    //  zero/engine.h:984-990; a caller of this boundary might, and would get uncapped logits without a word)
    if (w.softcap > 0.0f && cur_T_ > 8)
      throw std::logic_error(std::string("matmul ") + name + ": a matrix with a logit soft cap over more than 8 token rows (only the GEMVs cap)");
    q2_nocap_ = cap;
    q2_fuse_ = q2mm_ && !fuse_off && !q2_nofuse_ && cur_T_ <= 4;
    q2_fused_ = false;
    try {
      matmul1(name, w, Mp, C, ldc, c_off, acc, act32);
    } catch (...) {
      q2_fuse_ = false;
      q2_nocap_ = false;
      throw;
    }
    q2_fuse_ = false;
    if (!q2mm_) return;
    if (!q2_fused_) {
      const cl_mem a = aq_, s = asc_, b = absum_;
      aq_ = aq2_; asc_ = asc2_; absum_ = absum2_;
      try {
        matmul1(name, w, Mp, C, ldc, c_off, 1, act32);
      } catch (...) {
        aq_ = a; asc_ = s; absum_ = b;
        q2_nocap_ = false;
        throw;
      }
      aq_ = a; asc_ = s; absum_ = b;
    }
    q2_nocap_ = false;
    if (cap) {
      cl_kernel k = kernel("ops", "", "softcap_rows");
      int ld = cur_T_ == 1 ? 0 : ldc, off = c_off, N = w.N;
      float cp = w.softcap;
      set_args(k, 0, C, ld, off, N, cp);
      size_t gws[2] = {((size_t)N + 255) / 256 * 256, (size_t)cur_T_}, lws[2] = {256, 1};
      run(name, k, 2, gws, lws);
    }
  }

  // The same matmul for callers that must not allocate device memory (code under HIP graph capture, serving loops,
  // harnesses that forbid it): no counterpart in the reference.  The only device memory a matmul uses beyond its inputs
  // and outputs is the short-chunk GEMM's workspace of partial tiles; here it is the library's static scratch array
  // (arcz_scratch.hip, ARCZ_SCRATCH_BYTES, its address taken once at arcz_init) instead of the engine's buffer, the same
  // kernels with the same arguments otherwise, so the result is the ordinary entry point's bit for bit.  A launch that
  // would need more than the array holds is refused.  Launches are not timed (events are allocations).  Every call on
  // a GPU shares that GPU's array: calls that overlap on one GPU race (the library has one stream, so its own do not).
  bool noalloc_ = false;
  void matmul_noalloc(const char* name, const GpuWeight& w, int Mp, cl_mem C, int ldc, int c_off, int acc, bool act32) {
    if (!arcz_scratch_mem()) throw std::runtime_error("matmul_noalloc: the static device scratch was not set up");
    noalloc_ = true;
    try {
      matmul(name, w, Mp, C, ldc, c_off, acc, act32);
    } catch (...) {
      noalloc_ = false;
      throw;
    }
    noalloc_ = false;
  }

  // rows per half wave of the one-token GEMV (the place of the reference's gemv1_rows, zero/engine.h:1119-1123)
  static int gemv1_rows(const GpuWeight& w) {
    static const int force = getenv("ARCZ_GROWS") ? atoi(getenv("ARCZ_GROWS")) : 0;
    if (force == 1 || force == 2 || force == 4) return force <= w.N ? force : 1;
    return w.N <= 4096 ? 1 : 2;
  }
  static int gemv_mt_rows(const GpuWeight& w) {
    static const int force = getenv("ARCZ_GROWS_MT") ? atoi(getenv("ARCZ_GROWS_MT")) : 0;
    if (force == 1 || force == 2) return force;
    return w.N <= 4096 ? 1 : 2;
  }

  // The LDS-staged GEMVs' -DSCHED: how the rows of a launch of `wgs` work-groups of `g` rows a pass are dealt out (the
  // kernels would work it out themselves, in their first microsecond).  Whole rounds << 10 | rows of the one shorter
  // pass that every work-group gets of the rows left over -- when that is at least half a pass; else whole passes for
  // the first work-groups -- and, for two matrices in one launch, whole rounds << 10 | work-groups with a pass more.
  // Bit 30: the weight stream is read with non-temporal loads -- measured to pay from about 40 MB of matrix on (one
  // token, us with / without: Q4_K 17408 x 5120 10.0 / 10.4, Q8_0 15.5 / 16.4; 8192 x 8192 8.6 / 8.5, 4096 x 4096
  // 4.7 / 4.55), but not for one token over rows of 128 lanes and more (Q4_K 5120 x 17408: 11.15 / 10.9; two tokens,
  // in work-groups of 512: 12.65 / 13.2).  ARCZ_GEMV_NT=0 / 1: never / always.
  // `short_tail`: the rows left over go out as one short pass a work-group (one and two tokens of the types decoded
  // without a table -- GemvLds<QT>::short_tail: Q4_K one token 17408 x 5120 on 256 work-groups, 4 rows each, 10.6 ->
  // 10.5 us; Q6_K on 512, 2 rows each, 15.9 -> 14.8); otherwise as whole passes for the first work-groups (a short pass
  // still issues a whole pass's loads and takes a whole pass's time in the kernels bound by their arithmetic: IQ3_XXS
  // 12.1 -> 12.4 us, Q4_K four tokens 18.6 -> 20.8 with it).
  static int gemv_sched(int rows, int g, size_t wgs, bool two_matrices, size_t bytes, bool long_rows_one_token,
                        bool short_tail = false) {
    static const int nt_env = getenv("ARCZ_GEMV_NT") ? atoi(getenv("ARCZ_GEMV_NT")) : -1;
    const bool nt = nt_env >= 0 ? nt_env != 0 : bytes >= ((size_t)40 << 20) && !long_rows_one_token;
    const int ntb = nt ? 1 << 30 : 0;
    const int nw = (int)wgs;
    if (two_matrices) {
      const int npass = (rows + g - 1) / g;
      return ((npass / nw) << 10) | (npass % nw) | ntb;
    }
    const int full = rows / (g * nw);
    int tail = (rows - full * g * nw + nw - 1) / nw;
    if (!short_tail || tail == 0) tail = g;
    return (full << 10) | tail | ntb;
  }

  void matmul1(const char* name, const GpuWeight& w, int Mp, cl_mem C, int ldc, int c_off, int acc, bool act32) {
    if (!w.raw) throw std::runtime_error(std::string("matmul ") + name + ": the weight is not loaded");
    if (cur_T_ <= 0 || w.K != cur_K_ || Mp != cur_Mp_)
      throw std::runtime_error(std::string("matmul ") + name + ": the activations hold " + std::to_string(cur_Mp_) + " x " +
                               std::to_string(cur_K_) + ", the matrix takes " + std::to_string(Mp) + " x " + std::to_string(w.K));
    if (acc < 0 || acc > 2) throw std::runtime_error(std::string("matmul ") + name + ": accumulate mode");
    const int rows_out = cur_T_ > 8 ? Mp : cur_T_;
    if (c_off < 0 || (cur_T_ > 1 && c_off + w.N > ldc) ||
        arcz_mem_size(C) < ((size_t)(rows_out - 1) * (cur_T_ == 1 ? 0 : ldc) + c_off + w.N) * 4)
      throw std::runtime_error(std::string("matmul ") + name + ": the output does not fit C");
    int a = acc;
    cl_mem tabs = tabs_;  // (the reference's codebook tables; IQ3_S's kernels read theirs from it)
    // A few tokens, any weight type: the matrix-vector form on the matrix pipe (gemv_mm; it
    // takes K in slices of the tokens that fit LDS).  It takes 9-16 tokens in chunks of 16 rows (what the reference pads
    // them to, zero/engine.h:522; the rows from T on come out as zeros, as the GEMM writes them: Q4_K 21 against 95 us at
    // 17408 x 5120), and 3-8 tokens where it is the faster one: from 5 on always (us at the settled clock, 8 tokens,
    // against the dot-product kernels, 17408 x 5120: Q4_K 20.8 / 27.6, Q5_K 21.5 / 30.5, Q6_K 31.0 / 33.1, Q8_0 23.7 /
    // 31.4, Q4_0 20.2 / 27.7, IQ4_XS 23.4 / 31.0, IQ3_S 26.4 / 32.9; with 4 tokens 20.5 / 18.9, 21.4 / 20.7, 30.8 / 23.2, 23.6 / 20.1,
    // 20.4 / 17.1, 23.3 / 20.0: not taken; ARCZ_GEMV_MM_MIN: the first count it takes), 3 and 4 when the tokens do not
    // fit the LDS of the dot-product kernels (5120 x 17408, 4 tokens: Q4_K 34 against 88 us, Q5_K 42 against 97).  Not
    // with two-pass inputs (their second half goes through the kernels below).  ARCZ_GEMV_MM=0: off.
    static const bool mm_off = getenv("ARCZ_GEMV_MM") && atoi(getenv("ARCZ_GEMV_MM")) == 0;
    const bool mm_type = w.type == GGML_Q4_K || w.type == GGML_Q5_K || w.type == GGML_Q6_K || w.type == GGML_Q8_0 ||
                         w.type == GGML_Q4_0 || w.type == GGML_IQ4_XS || w.type == GGML_IQ3_S || w.type == GGML_IQ4_NL ||
                         w.type == GGML_MXFP4 || w.type == GGML_Q3_K || w.type == GGML_IQ3_XXS;
    const bool mm_ok = !mm_off && !q2mm_ && mm_type && a <= 1 && w.softcap <= 0.0f;  // (gemv_mm has no soft cap)
    auto gemv_mm = [&] {
      int N = w.N, K = w.K, M = Mp, T = cur_T_;
      rd_bytes += raw_bytes(w);
      cl_kernel k = kernel("decode", "-DQT=" + std::to_string(w.type), "gemv_mm");
      const size_t groups = (size_t)(N + 15) / 16, cus = (size_t)arcz_device_cus();
      // Rows longer than the tokens' LDS holds (slices of sb_max superblocks): K is shared out over `ny` work-groups
      // per run of groups, each staging its piece of the tokens once, and gemv_mm_reduce adds the pieces -- inside one
      // work-group the slices are staged one after the other, and 320 groups on 256 work-groups leave a quarter of them
      // two groups and the rest one (8 tokens, us: 5120 x 17408 Q4_K 34.4 -> 22.6, Q6_K 58.0 -> 32.1, Q8_0 34.4 -> 25.7;
      // 17408 x 17408 Q4_K 60.7 -> 44.9; 40960 x 8192 Q4_K 60.9 -> 46.7, Q8_0 69.1 -> 72.5).  Up to 12 groups a compute
      // unit (ARCZ_GEMV_MM_SK=n: n, 0: never); beyond that, and when the workspace is not to be had, the kernel walks
      // the slices itself.
      static const int sk_env = getenv("ARCZ_GEMV_MM_SK") ? atoi(getenv("ARCZ_GEMV_MM_SK")) : -1;
      static const bool sk_off = sk_env == 0;
      const size_t sk_groups = (size_t)(sk_env > 0 ? sk_env : 12) * cus;
      const int nsb = K / 256;
      const int sb_max = w.type == GGML_Q6_K ? 20 : w.type == GGML_Q5_K || w.type == GGML_IQ3_S || w.type == GGML_Q3_K || w.type == GGML_IQ3_XXS ? 22 : 24;  // (the kernels' MmT<QT>::SB)
      const int ny = (nsb + sb_max - 1) / sb_max;
      const size_t need = (size_t)ny * 16 * N * 4;
      cl_mem ws = noalloc_ ? arcz_scratch_mem() : sk_ws_;
      if (!sk_off && ny >= 2 && groups <= sk_groups && (!noalloc_ || need <= arcz_mem_size(ws))) {
        if (!noalloc_ && need > sk_ws_bytes_) {
          if (sk_ws_) release(sk_ws_);
          sk_ws_ = nullptr;
          sk_ws_bytes_ = 0;
          sk_ws_ = buf(need);
          sk_ws_bytes_ = need;
          ws = sk_ws_;
        }
        int zero = 0, ldw = N, s1 = nsb;
        set_args(k, 0, w.raw, N, K, tabs, aq_, asc_, absum_, M, T, ws, ldw, zero, zero, zero, s1);
        size_t g2[2] = {std::min<size_t>(groups, std::max<size_t>(cus / (size_t)ny, 1)) * 512, (size_t)ny}, l2[2] = {512, 1};
        run(name, k, 2, g2, l2);
        cl_kernel kr = kernel("decode", "", "gemv_mm_reduce");
        int rows = T > 8 ? 16 : T, nyy = ny;
        set_args(kr, 0, ws, nyy, C, rows, N, ldc, c_off, a);
        size_t g3 = ((size_t)rows * N + 255) / 256 * 256, l3 = 256;
        run(name, kr, 1, &g3, &l3);
        return;
      }
      size_t g1 = std::min<size_t>(groups, cus) * 512, l1 = 512;
      set_args(k, 0, w.raw, N, K, tabs, aq_, asc_, absum_, M, T, C, ldc, c_off, a, 0, K / 256);
      run(name, k, 1, &g1, &l1);
    };
    if (mm_ok && cur_T_ >= 9 && cur_T_ <= 16 && Mp == 16) {
      gemv_mm();
      return;
    }
    if (cur_T_ >= 1 && cur_T_ <= 8) {
      if (a > 1) throw std::logic_error(std::string("GEMV with a fused epilogue: ") + name);
      int N = w.N, K = w.K, M = Mp, T = cur_T_;
      rd_bytes += raw_bytes(w);
      // The main kernels stage the tokens' activations in LDS (gemv / gemv_mt); when T tokens of K values do not fit
      // the 64 KiB a launch may ask for, the kernels that read them from global memory take over (gemv_v / gemv_mt_v).
      const int ups = w.type == GGML_Q8_0 ? 16 : 8, units = K / 256 * ups;
      // (a token's bytes in LDS: 16 values and a scale per unit and part; Q4_K / Q5_K: the scale times the block sum
      //  beside it; Q6_K in the one-token kernel: the 16 values' sum)
      auto tokb = [&](int slots) {
        const bool wide = w.type == GGML_Q4_K || w.type == GGML_Q5_K ||
                          ((w.type == GGML_Q6_K || w.type == GGML_Q3_K) && slots == 1);
        return (w.type == GGML_Q8_0 ? 1 : 2) * units * (16 + (wide ? 8 : 4));
      };
      static const int force_v = getenv("ARCZ_GEMV_V") ? atoi(getenv("ARCZ_GEMV_V")) : 0;
      // lanes per row: the fewest of 32 / 64 / 128 / 256 that leave a lane at most 6 sixteen-byte units of a row
      static const int force_lpr = getenv("ARCZ_GEMV_LPR") ? atoi(getenv("ARCZ_GEMV_LPR")) : 0;
      int lpr = 0;
      for (int l : {32, 64, 128, 256})
        if (!lpr && (units + l - 1) / l <= 6 && (!force_lpr || l == force_lpr)) lpr = l;
      // Rows of 128 or 256 lanes, two tokens: work-groups of 512 threads, one a compute unit, stage the tokens once per
      // compute unit instead of twice (5120 x 17408 Q4_K: 15.0 -> 14.4 us; one token: 11.9 -> 12.2, so not taken there;
      // ARCZ_GEMV_BT=256: never, =512: for one token too)
      static const int bt_env = getenv("ARCZ_GEMV_BT") ? atoi(getenv("ARCZ_GEMV_BT")) : 0;
      const int bt = lpr >= 128 && (T == 2 || (T == 1 && bt_env == 512)) && !q2_fuse_ && bt_env != 256 ? 512 : 256;
      const int g = lpr ? bt / lpr : 1, wpr = lpr > 64 ? lpr / 64 : 1;
      // the kernel's token slots: T rounded up, or -- both halves of two-pass inputs in one launch -- 2 T rounded up
      auto lds_of = [&](int slots) { return (size_t)slots * tokb(slots) + (wpr > 1 ? (size_t)16 * g * wpr * slots * 4 : 0); };  // (16: the kernels' GEMV_FLUSH)
      const int tb2 = T == 1 ? 2 : T == 2 ? 4 : 8;
      const bool q2f = q2_fuse_ && T <= 4 && lpr && lds_of(tb2) <= (w.type == GGML_IQ3_S || w.type == GGML_IQ3_XXS ? 65536 - 2048 : 65536);
      const int tbl = q2f ? tb2 : T <= 2 ? T : T <= 4 ? 4 : 8;
      const size_t lds = lds_of(tbl);
      // (IQ3_S: 2 KiB of the work-group's LDS hold the codebook)
      const size_t lds_max = w.type == GGML_IQ3_S || w.type == GGML_IQ3_XXS ? 65536 - 2048 : 65536;
      const bool fits = !force_v && lpr && lds <= lds_max;
      static const int mm_min = getenv("ARCZ_GEMV_MM_MIN") ? atoi(getenv("ARCZ_GEMV_MM_MIN")) : 5;
      if (mm_ok && T >= 3 && (T >= mm_min || !fits)) {
        rd_bytes -= raw_bytes(w);  // (counted by gemv_mm)
        gemv_mm();
        return;
      }
      if (fits) {
        const int pf = (units + lpr - 1) / lpr, tb = tbl;
        // one round of resident work-groups, passes of rows dealt to them in turn (ARCZ_GEMV_WPC: work-groups per
        // compute unit).  One token: one work-group a compute unit -- measured at the settled clock against two, us per
        // launch: Q4_K 17408 x 5120 10.56 / 10.66, 5120 x 17408 10.93 / 11.84, 4096 x 4096 4.25 / 4.69, 1024 x 5120
        // 5.13 / 5.74, Q6_K 151936 x 5120 107.7 / 111.5, Q5_K 13.11 / 13.42 -- except for the codebook types, whose
        // decode wants the second work-group's waves (IQ4_XS 13.24 / 12.95).  More tokens: two (four tokens at
        // 17408 x 5120: 20.2 against 25.7 with one; three or four per unit are slower everywhere).
        static const int wpc_env = getenv("ARCZ_GEMV_WPC") ? atoi(getenv("ARCZ_GEMV_WPC")) : 0;
        static const int wgs_env = getenv("ARCZ_GEMV_WGS") ? atoi(getenv("ARCZ_GEMV_WGS")) : 0;
        const bool codebook = w.type == GGML_IQ4_XS || w.type == GGML_IQ3_S || w.type == GGML_IQ4_NL || w.type == GGML_MXFP4 ||
                              w.type == GGML_IQ3_XXS;
        // (Q6_K, one token, since its kernel takes the - 32 off the sums: two work-groups a unit are ahead on matrices
        //  of layer size -- 17408 x 5120 16.4 -> 15.9 us, 5120 x 17408 16.3 -> 15.9, 8192 x 8192 12.8 -> 12.3 -- and
        //  behind on the 151936 x 5120 output head, 106.3 -> 110.3)
        // (Q3_K, one token: two everywhere -- 17408 x 5120 11.6 -> 10.7 us, 5120 x 17408 13.5 -> 11.3, 4096 x 4096
        //  5.0 -> 4.6; Q5_K and Q8_0 measured beside it stay at one: 12.8 -> 13.1 and 16.9 -> 17.1)
        const bool q6_mid = (w.type == GGML_Q6_K && tb == 1 && (size_t)N * (size_t)K <= ((size_t)1 << 28)) ||
                            (w.type == GGML_Q3_K && tb == 1);
        const int wpc = wpc_env > 0 ? wpc_env : bt == 512 || (tb == 1 && !codebook && !q6_mid) ? 1 : 2;
        size_t wgs = std::min<size_t>((size_t)(N + g - 1) / g, (size_t)arcz_device_cus() * wpc);
        if (wgs_env > 0) wgs = std::min<size_t>((size_t)(N + g - 1) / g, (size_t)wgs_env);
        const std::string defs = "-DQT=" + std::to_string(w.type) + " -DLPR=" + std::to_string(lpr) + " -DPF=" +
                                 std::to_string(pf) + (tb > 1 ? " -DTB=" + std::to_string(tb) : std::string()) +
                                 (bt == 512 ? " -DBT=512" : "") + " -DLDS=" +
                                 std::to_string(lds) +
                                 (q2f ? " -DQ2_AQ=" + std::to_string(q2_aq_) + " -DQ2_SC=" + std::to_string(q2_sc_ / 4) : std::string()) +
                                 head_defs(w) + " -DSCHED=" + std::to_string(gemv_sched(N, g, wgs, false, raw_bytes(w), lpr >= 128 && tb == 1 && bt == 256, !codebook && tb <= 2));
        cl_kernel k = kernel("decode", defs, tb == 1 ? "gemv" : "gemv_mt");
        int ld1 = T == 1 ? 0 : ldc;  // (one token: C is the row itself)
        if (tb == 1) set_args(k, 0, w.raw, N, K, tabs, aq_, asc_, absum_, M, C, c_off, a);
        else set_args(k, 0, w.raw, N, K, tabs, aq_, asc_, absum_, M, T, C, ld1, c_off, a);
        q2_fused_ = q2f;
        size_t g1 = wgs * (size_t)bt, l1 = (size_t)bt;
        run(name, k, 1, &g1, &l1);
        return;
      }
      const int gr = T == 1 ? gemv1_rows(w) : gemv_mt_rows(w);
      const std::string defs = "-DQT=" + std::to_string(w.type) + " -DGROWS=" + std::to_string(gr) +
                               (T > 1 ? " -DTB=" + std::to_string(T) : std::string()) + head_defs(w);
      cl_kernel k = kernel("decode", defs, T == 1 ? "gemv_v" : "gemv_mt_v");
      if (T == 1) set_args(k, 0, w.raw, N, K, tabs, aq_, asc_, absum_, M, C, c_off, a);
      else set_args(k, 0, w.raw, N, K, tabs, aq_, asc_, absum_, M, T, C, ldc, c_off, a);
      size_t g1 = ((size_t)(N + gr - 1) / gr * 32 + 255) / 256 * 256, l1 = 256;
      run(name, k, 1, &g1, &l1);
      return;
    }
    gemm_dense(name, w, Mp, C, ldc, c_off, a);
  }

  // One token: the FFN's gate and up GEMVs in one launch (zero/engine.h:1124-1146, the kernel's -DGU2 form): rows
  // [0, F) of gate at C and [0, F) of up at C + F, every row by the lanes and arithmetic of its own launch, bit for bit.
  // On this machine a launch of 50 MB spends about 4 of its 10 us filling and draining the chip; one launch of twice
  // the bytes pays that once.  false: not taken (the caller runs the two launches): more than one token, two-pass
  // inputs, matrices that differ in type or shape, rows too long for the LDS-staged kernel, or F not a multiple of the
  // rows of a pass.  ARCZ_GEMV_GU=0: never taken.
  bool gemv_gu(const GpuWeight& g, const GpuWeight& u, int Mp, cl_mem C) {
    static const bool off = getenv("ARCZ_GEMV_GU") && atoi(getenv("ARCZ_GEMV_GU")) == 0;
    if (off || cur_T_ != 1 || q2mm_ || !cur_act32_ || !g.raw || !u.raw || g.type != u.type || g.N != u.N || g.K != u.K)
      return false;
    if (g.K != cur_K_ || Mp != cur_Mp_)
      throw std::runtime_error("gemv_gu: the activations hold " + std::to_string(cur_Mp_) + " x " + std::to_string(cur_K_) +
                               ", the matrices take " + std::to_string(Mp) + " x " + std::to_string(g.K));
    const int N = g.N, K = g.K;
    const int ups = g.type == GGML_Q8_0 ? 16 : 8, units = K / 256 * ups;
    const int tok_bytes = (g.type == GGML_Q8_0 ? 1 : 2) * units * (16 + (g.type == GGML_Q4_K || g.type == GGML_Q5_K || g.type == GGML_Q6_K || g.type == GGML_Q3_K ? 8 : 4));
    int lpr = 0;
    for (int l : {32, 64, 128, 256})
      if (!lpr && (units + l - 1) / l <= 6) lpr = l;
    if (!lpr) return false;
    const int gr = 256 / lpr, wpr = lpr > 64 ? lpr / 64 : 1;
    const size_t lds = (size_t)tok_bytes + (wpr > 1 ? (size_t)16 * gr * wpr * 4 : 0);
    if (lds > (g.type == GGML_IQ3_S || g.type == GGML_IQ3_XXS ? 65536u - 2048u : 65536u) || N % gr) return false;
    if (arcz_mem_size(C) < (size_t)2 * N * 4) throw std::runtime_error("gemv_gu: the output does not fit C");
    rd_bytes += raw_bytes(g) + raw_bytes(u);
    const int pf = (units + lpr - 1) / lpr;
    static const int gu_wpc = getenv("ARCZ_GEMV_GU_WPC") ? atoi(getenv("ARCZ_GEMV_GU_WPC")) : 1;  // (17.6 against 18.2 us with two)
    const size_t wgs = std::min<size_t>((size_t)2 * N / gr, (size_t)arcz_device_cus() * gu_wpc);
    const std::string defs = "-DQT=" + std::to_string(g.type) + " -DLPR=" + std::to_string(lpr) + " -DPF=" + std::to_string(pf) +
                             " -DLDS=" + std::to_string(lds) + " -DGU2 -DSCHED=" +
                             std::to_string(gemv_sched(2 * N, gr, wgs, true, raw_bytes(g) + raw_bytes(u), lpr >= 128));
    cl_kernel k = kernel("decode", defs, "gemv");
    cl_mem tabs = tabs_;
    int NN = N, KK = K, M = Mp, c_off = 0, a = 0;
    set_args(k, 0, g.raw, NN, KK, tabs, aq_, asc_, absum_, M, C, c_off, a, u.raw);
    size_t g1 = wgs * 256, l1 = 256;
    run("gemm_gate_up", k, 1, &g1, &l1);
    return true;
  }

  // The prefill GEMM (zero/engine.h:1205-1250).  Token rows come in whole tiles (the reference pads a chunk to 128
  // rows from 128 tokens on, :521-522).
  // Workspace of the short-chunk GEMM's partial tiles, [slices][Mp][N] f32: allocated with the engine (only a forced
  // piece count, ARCZ_Q4_SPLITK=n read when the engine is made, can outgrow it; then it is replaced by a larger one).
  cl_mem sk_ws_ = nullptr;
  size_t sk_ws_bytes_ = 0;
  int sk_force_ = -1;  // ARCZ_Q4_SPLITK: 0 = never share K out, n >= 2: n pieces, -1 = the rule below
  bool moe_dec_off_ = false, moe_fuse_off_ = false, moe_qfuse_off_ = false;  // ARCZ_MOE_DECODE / _FUSE / _QFUSE = 0
  int moe_dec_max_ = 16, moe_tmd_ = 0;                                      // ARCZ_MOE_DECODE_MAX, ARCZ_MOE_TMD
  int q4_wm_ = 0, q4_wm_min_ = 2048;                                        // ARCZ_Q4_WM (0: by rule), ARCZ_Q4_WM_MIN (of =4)
  bool moe_pre_ = true;                                                     // ARCZ_MOE_PRE (0: off)
  // (The gate / up tile kernel on ready-made scale vectors runs in steps of 64 values, three work-groups a compute unit:
  // 0.401 -> 0.369 ms at 4096 tokens against the same in steps of 128 at two a unit, same bits.  The down projection's
  // kernel in that form -- 121 registers, four work-groups a compute unit -- was built and measured equal to its
  // three-a-unit form in steps of 128: 0.2275 against 0.2255 ms; not kept.)
  void gemm_dense(const char* name, const GpuWeight& w0, int Mp, cl_mem C, int ldc, int c_off, int a) {
    const GpuWeight w = gemm_form(name, w0);
    int M = Mp, N = w.N, K = w.K;
    // Any type, a chunk so short that its tiles are fewer than two per compute unit: K is shared out over `ny`
    // work-groups per tile, which store partial tiles in a workspace, and splitk_reduce adds the slices in order (the
    // same bits on every run) and applies c_off and the accumulate mode.  One work-group needs 75 us for K = 5120, so
    // 64 tokens x 17408 rows took 100 us whatever the tile; now 136 tiles x 3 pieces, 42 us (128 tokens: 101 -> 71 us;
    // Q8_0 4096 x 4096: 64 tokens 41 -> 19 us, 256 tokens 44 -> 35 us).  ARCZ_Q4_SPLITK=0: off, =n: n pieces.
    if (sk_force_ != 0) {
      // (tiles of 64 tokens up to 64 tokens, else of 128: the pieces of all tiles together must fit the resident slots,
      //  two work-groups per compute unit: one more piece than fits costs a whole second round)
      // (Q8_0, Q6_K: their dense kernels' 64-token tiles; IQ4_XS: the register-staged body's 128-token tiles)
      const bool q45 = w.type == GGML_Q4_K || w.type == GGML_Q5_K;
      const int tm = w.type == GGML_Q8_0 || w.type == GGML_Q6_K ? 64 : q45 ? (Mp <= 64 ? 64 : 128) : 128;
      const int bm = tm == 64 && q45 && Mp <= 32 ? 32 : tm;  // (Q4_K / Q5_K, at most 32 rows: the one-slot-tile kernel)
      // (the one-slot-tile kernel is light enough for three work-groups a compute unit: 17408 x 5120, 32 tokens, 3 pieces
      //  of K 30.0 us, 5 pieces 28.3)
      const size_t tiles64 = (size_t)((Mp + tm - 1) / tm) * ((N + 127) / 128), slots = (bm == 32 ? 3 : 2) * (size_t)arcz_device_cus();
      const int nsb = K / 256;
      const int sk_force = sk_force_;
      int ny = (int)std::min<size_t>({(size_t)8, (size_t)nsb / 2, slots / std::max<size_t>(tiles64, 1)});
      if (sk_force >= 2) ny = std::min(sk_force, nsb);
      // (from three pieces on: with two, 256 tiles of Q8_0 4096 x 4096 x 512 went from 50 to 54 us, the reduce included)
      if (ny >= 3 || (sk_force >= 2 && ny >= 2)) {
        const size_t need = (size_t)ny * Mp * N * 4;
        cl_mem ws = sk_ws_;
        if (noalloc_) {
          ws = arcz_scratch_mem();
          if (need > arcz_mem_size(ws))
            throw std::runtime_error(std::string("matmul_noalloc ") + name + ": " + std::to_string(ny) + " partial tiles of " +
                                     std::to_string(Mp) + " x " + std::to_string(N) + " need " + std::to_string(need) +
                                     " bytes of workspace, the static scratch holds " + std::to_string(arcz_mem_size(ws)));
        } else if (need > sk_ws_bytes_) {
          if (sk_ws_) release(sk_ws_);
          sk_ws_ = nullptr;
          sk_ws_bytes_ = 0;
          sk_ws_ = buf(need);
          sk_ws_bytes_ = need;
          ws = sk_ws_;
        }
        cl_kernel k = kernel("gemm", std::string("-DQTYPE=") + std::to_string(w.type) + " -DACT32 -DBM=" + std::to_string(bm) +
                                         " -DBN=128 -DSPLITK" + (w.half_d ? " -DHDS=" + std::to_string(w.half_d) : std::string()), "gemm");
        cl_mem unused = nullptr;
        int zero = 0, one = 1, ldw = N, s1 = nsb;
        set_args(k, 0, w.raw, unused, aq_, asc_, absum_, ws, M, N, K, ldw, zero, zero, one, zero, s1);
        size_t gws[2] = {tiles64 * 256, (size_t)ny}, lws[2] = {256, 1};
        run(name, k, 2, gws, lws);
        cl_kernel r = kernel("gemm", "", "splitk_reduce");
        int nyy = ny;
        set_args(r, 0, ws, nyy, C, M, N, ldc, c_off, a);
        size_t g1 = ((size_t)M * N + 255) / 256 * 256, l1 = 256;
        run(name, r, 1, &g1, &l1);
        return;
      }
    }
    // tiles of 128 tokens x 128 rows (or 64 x 256) for Q4_K, 64 x 128 for Q6_K and Q8_0 (whose 64-token kernel measured 1.9 x the
    // 128-token one at 17408 x 5120 x 8192 and 3 x at 4096 x 4096 x 512; ARCZ_Q8_BM=128 brings the latter back)
    static const int q8_bm = getenv("ARCZ_Q8_BM") ? atoi(getenv("ARCZ_Q8_BM")) : 0;
    const bool q8_small = w.type == GGML_Q8_0 && q8_bm != 128;
    static const int q4_bm = getenv("ARCZ_Q4_BM") ? atoi(getenv("ARCZ_Q4_BM")) : 0;
    // Q4_K: tiles of 64 tokens x 256 rows (the same work per work-group and the same rate as 128 x 128) when the last
    // 128 token rows of a short chunk are at most half full (ARCZ_Q4_BM=64 always, =128 never)
    const bool q4_wide = w.type == GGML_Q4_K && (q4_bm == 64 || (q4_bm == 0 && Mp <= 1024 && ((Mp - 1) & 127) < 64));
    // Q4_K, few tokens: 64 x 128 tiles when the larger ones would leave compute units idle (ARCZ_Q4_BN=128 always)
    static const int q4_bn = getenv("ARCZ_Q4_BN") ? atoi(getenv("ARCZ_Q4_BN")) : 0;
    static const int q4_small_max = getenv("ARCZ_Q4_SMALL") ? atoi(getenv("ARCZ_Q4_SMALL")) : 0;
    const bool q4_small = w.type == GGML_Q4_K && (q4_bn == 128 || (q4_bn == 0 && Mp <= q4_small_max));
    // Q4_K / Q5_K in 128 x 128 tiles: the token side's scale vectors ready-made (-DAU; ARCZ_Q4_AU=0: formed in the kernel)
    static const int q4_au = getenv("ARCZ_Q4_AU") ? atoi(getenv("ARCZ_Q4_AU")) : 3;
    const bool au = q4_au && (w.type == GGML_Q4_K || w.type == GGML_Q5_K) && !q4_wide && !q4_small && M % 4 == 0;
    // ... and the row side's too (-DAU=2), written in front of the launch (8 bytes per 32 weights: 22 MB, about 8 us,
    // for 17408 x 5120; pays from the shortest chunks this path takes: ARCZ_Q4_AU=1 never, ARCZ_Q4_AU2_MIN=n from n
    // token rows on)
    static const int au2_min = getenv("ARCZ_Q4_AU2_MIN") ? atoi(getenv("ARCZ_Q4_AU2_MIN")) : 256;
    const bool au2 = au && q4_au >= 2 && Mp >= au2_min && N % 4 == 0 && (size_t)N * (K / 32) * 21 + 4096 <= wsv_bytes_;
    // ... and, Q4_K, the min term's operands as bf16 pieces (-DAU=3: 20 bytes per block and row to write, 56 MB,
    // about 15 us, for 17408 x 5120; us per launch at that shape against the -DAU=2 form, both with their pre-passes:
    // 512 tokens 199 / 210, 1024 313 / 331, 2048 545 / 577, 8192 2062 / 2121; ARCZ_Q4_AU=2 never, ARCZ_Q4_AU3_MIN=n
    // from n token rows on)
    static const int au3_min = getenv("ARCZ_Q4_AU3_MIN") ? atoi(getenv("ARCZ_Q4_AU3_MIN")) : 256;
    const bool au3 = au2 && q4_au >= 3 && w.type == GGML_Q4_K && Mp >= au3_min;
    // ... and, when the chunk's activation scales are per 256 values (act32 = 0: asc_ is their per-32 expansion), the
    // form that adds a superblock's block sums up as integers (-DAU=4; ARCZ_Q4_A256=0: the per-32 form on the expansion)
    static const bool a256_off = getenv("ARCZ_Q4_A256") && atoi(getenv("ARCZ_Q4_A256")) == 0;
    const bool au4 = au3 && a256_ && !a256_off;
    // ... in tiles of 256 tokens x 128 rows, work-groups of 512 threads (ARCZ_Q4_WM=4, read when the engine is made; from
    // ARCZ_Q4_WM_MIN token rows on).  Not the default: ms per launch at 17408 x 5120 against the 128 x 128 tiles, same
    // box, 8192 tokens 2.13 / 2.12, 4096 1.107 / 1.06, 2048 0.613 / 0.552 -- one work-group of 8 waves a compute unit
    // meets at one barrier where two of 4 waves overlap each other's waits, and 256-token tiles fill the last round worse.
    const bool wm4 = au3 && !au4 && q4_wm_ == 4 && Mp >= q4_wm_min_;
    // ... or in tiles of 64 tokens x 128 rows on f32 scale vectors, work-groups of 168 registers, three a compute unit.
    // In the steady state the smaller tile loses (8192 tokens at 17408 x 5120: 681 against 727 TOP/s: each step's
    // row-side traffic and scale tiles serve half the products), but a short chunk is a few rounds of work-groups and
    // which tile fills its last round better decides: ms per launch, 64 x 128 against 128 x 128, at 17408 x 5120: 256
    // tokens 0.108 / 0.132, 384 0.143 / 0.132, 512 0.170 / 0.193, 768 0.230 / 0.243, 1024 0.291 / 0.302, 2048 0.550 /
    // 0.535; 5120 x 17408 x 1024 0.331 / 0.393, x 1536 0.449 / 0.406; 8192 x 8192 x 768 0.166 / 0.194, x 1024 0.221 /
    // 0.204.  The rule prices both in rounds of the large tiles (two work-groups a compute unit): a full round of the
    // small ones (three a unit, 3/4 of the work at 681 / 727 of the rate) 0.8; a last round in which every compute unit
    // has at most one large tile 0.5, else 1; at most one small tile 0.30, at most two 0.48, else 0.8 -- fitted to a
    // sweep of nine matrices x twelve chunk lengths, where it picks the slower tile by more than 2 % in one case of 103.
    // ARCZ_Q4_WM=1 always, =2 never.
    bool t64 = au2 && !au4 && w.type == GGML_Q4_K && (q4_wm_ == 1 || q4_wm_ == 0);
    if (t64 && q4_wm_ == 0) {
      const size_t cus = (size_t)arcz_device_cus(), nt = (size_t)(N + 127) / 128;
      const size_t t128 = (size_t)((Mp + 127) / 128) * nt, s128 = 2 * cus, r128 = t128 % s128;
      const size_t t64n = (size_t)((Mp + 63) / 64) * nt, s64 = 3 * cus, r64 = t64n % s64;
      const double c128 = (double)(t128 / s128) + (r128 == 0 ? 0.0 : 2 * r128 <= s128 ? 0.5 : 1.0);
      const double c64 = 0.8 * (double)(t64n / s64) + (r64 == 0 ? 0.0 : 3 * r64 <= s64 ? 0.30 : 3 * r64 <= 2 * s64 ? 0.48 : 0.8);
      t64 = c64 < 0.97 * c128;
    }
    if (t64) {
      cl_kernel ku = kernel("ops", "", "act_usum");
      set_args(ku, 0, asc_, absum_, M, au_);
      size_t g2[2] = {(size_t)(M + 255) / 256 * 256, (size_t)(K / 32)}, l2[2] = {256, 1};
      run("act_usum", ku, 2, g2, l2);
      cl_kernel kw = kernel("ops", "", "q4k_wscales");
      size_t hdr = planes_q4k((size_t)N, K / 256).hdr;
      int NN = N, nsb2 = K / 256;
      set_args(kw, 0, w.raw, hdr, NN, nsb2, wsv_);
      size_t g3[2] = {(size_t)(N + 255) / 256 * 256, (size_t)(K / 256)};
      run("q4k_wscales", kw, 2, g3, l2);
      cl_kernel k = kernel("gemm", "-DQTYPE=12 -DACT32 -DBM=64 -DBN=128 -DPRE64=1", "gemm");
      int rgroup = 1, s0 = 0, s1 = K / 256;
      set_args(k, 0, w.raw, au_, aq_, asc_, wsv_, C, M, N, K, ldc, c_off, a, rgroup, s0, s1);
      size_t gws[1] = {(size_t)((Mp + 63) / 64) * ((N + 127) / 128) * 256}, lws[1] = {256};
      run(name, k, 1, gws, lws);
      return;
    }
    cl_kernel k = wm4       ? kernel("gemm", "-DQTYPE=12 -DACT32 -DAU=3 -DWM=4", "gemm")
                  : q8_small ? kernel("gemm", "-DQTYPE=8 -DACT32 -DBM=64", "gemm")
                  : q4_small ? kernel("gemm", "-DQTYPE=12 -DACT32 -DBM=64 -DBN=128", "gemm")
                  : q4_wide ? kernel("gemm", "-DQTYPE=12 -DACT32 -DBM=64", "gemm")
                  : au      ? kernel("gemm", "-DQTYPE=" + std::to_string(w.type) + (au4 ? " -DACT32 -DAU=4" : au3 ? " -DACT32 -DAU=3" : au2 ? " -DACT32 -DAU=2" : " -DACT32 -DAU"), "gemm")
                            : gemm_kernel(w.type, false, 0, w.half_d);
    // (ARCZ_GEMM_SPLIT: superblocks per split-K piece, 0 = one pass, the default here: a work-group keeps its sums in
    //  registers over the whole of K.  The reference splits rows longer than 8192 into 17-superblock pieces for its
    //  cache, zero/engine.h:1236-1250; pieces after the first accumulate into C and are not bit-identical to one pass.)
    static const int sk_sb = getenv("ARCZ_GEMM_SPLIT") ? std::max(0, atoi(getenv("ARCZ_GEMM_SPLIT"))) : 0;
    const int nsb = K / 256, splits = a != 2 && sk_sb > 0 ? (nsb + sk_sb - 1) / sk_sb : 1, rgroup = 1;
    cl_mem unused = nullptr;
    const int bm = wm4 ? 256 : w.type == GGML_Q6_K || q8_small || q4_wide || q4_small ? 64 : 128;  // token rows of a work-group's tile
    const int bn = q4_wide && !q4_small ? 256 : 128;
    const size_t tiles = (size_t)((Mp + bm - 1) / bm) * ((N + bn - 1) / bn);
    const size_t wg = wm4 ? 512 : 256;
    size_t gws[1] = {tiles * wg}, lws[1] = {wg};
    if (au) {
      cl_kernel ku = kernel("ops", "", au3 ? "act_usum_bf16" : "act_usum");
      set_args(ku, 0, asc_, absum_, M, au_);
      size_t g2[2] = {(size_t)(M + 255) / 256 * 256, (size_t)(K / 32)}, l2[2] = {256, 1};
      run("act_usum", ku, 2, g2, l2);
      unused = au_;
    }
    cl_mem sums = absum_;
    if (au2) {
      cl_kernel kw = kernel("ops", "", au4 ? "q4k_wscales_int" : au3 ? "q4k_wscales_bf16" : "q4k_wscales");
      size_t hdr = planes_q4k((size_t)N, K / 256).hdr;
      int NN = N, nsb2 = K / 256;
      set_args(kw, 0, w.raw, hdr, NN, nsb2, wsv_);
      size_t g2[2] = {(size_t)(N + 255) / 256 * 256, (size_t)(K / 256)}, l2[2] = {256, 1};
      run("q4k_wscales", kw, 2, g2, l2);
      sums = wsv_;
    }
    for (int sp = 0; sp < splits; ++sp) {
      int s0 = nsb * sp / splits, s1 = nsb * (sp + 1) / splits, ac = sp == 0 ? a : 1;
      set_args(k, 0, w.raw, unused, aq_, asc_, sums, C, M, N, K, ldc, c_off, ac, rgroup, s0, s1);
      run(name, k, 1, gws, lws);
    }
  }
  // (zero/engine_setup.h:384-420 gemm_kernel / moe_gemm_kernel)
  cl_kernel gemm_kernel(uint32_t qtype, bool tiles, int ne = 0, int half_d = 0) {
    std::string defs = "-DQTYPE=" + std::to_string(qtype) + " -DACT32";
    if (tiles) defs += " -DMOE_TILES -DNE=" + std::to_string(ne);
    if (half_d) defs += (tiles ? " -DHDT=" : " -DHD=") + std::to_string(half_d);
    return kernel("gemm", defs, "gemm");
  }

  // ---------------------------------------------------------------- mixture of experts (zero/engine_moe.h)
  struct MoeLayer {
    GpuWeight ex[3];  // gate, up [NE][F][E]; down [NE][E][F]
    int NE = 0, NU = 0, E = 0, F = 0;
    // the reference's routing variants (zero/engine_moe.h:99-101, zero/kernels/moe.cl:17-46): escale [NE] f32 -- each
    // chosen expert's weight times its scale (-DESCALE); ebias [NE] f32 + rscale -- the sqrt(softplus) scores chosen with
    // a bias (-DROUTE_DS -DRSCALE)
    cl_mem escale = nullptr, ebias = nullptr;
    float rscale = 1.0f;
    // Q4_K tensors (ARCZ_MOE_PRE=0 when the engine is made: none): the rows' scale vectors ws | v (q4k_wscales over the
    // tensor as one matrix of NE * rows: 8 bytes per 32 weights on top of the 18 of the planes), which the tile kernels
    // of a chunk of many tokens then take by DMA instead of unpacking the 6-bit scales per tile and step.  A layer of
    // 128 experts x 768 x 2048 at 4096 tokens: 0.80 -> 0.70 ms (gate / up 0.430 -> 0.375, down 0.256 -> 0.212: without
    // the scale registers both tile kernels fit three work-groups a compute unit) for 151 MB on top of the layer's 340.
    cl_mem wsv[3] = {nullptr, nullptr, nullptr};
    bool variant() const { return escale || ebias; }
    std::string route_defs() const {
      if (ebias) {
        char b[64];
        snprintf(b, sizeof b, " -DROUTE_DS -DRSCALE=%.9ef", rscale);
        return b;
      }
      return escale ? " -DESCALE" : "";
    }
  };
  void set_moe_routing(MoeLayer& L, const float* escale, const float* ebias, float rscale) {
    if (escale && ebias) throw std::runtime_error("set_moe_routing: expert scales and the biased routing do not combine");
    for (cl_mem* m : {&L.escale, &L.ebias})
      if (*m) { release(*m); *m = nullptr; }
    if (escale) L.escale = buf((size_t)L.NE * 4, escale);
    if (ebias) L.ebias = buf((size_t)L.NE * 4, ebias);
    L.rscale = rscale;
  }
  // buffers of the layer (zero/engine_alloc.h:109-159): sized for max_chunk tokens
  cl_mem mids_ = nullptr, mwts_ = nullptr, sgate_ = nullptr, mcount_ = nullptr, moffs_ = nullptr, mcursor_ = nullptr,
         mtiles_ = nullptr, mtstart_ = nullptr, stok_ = nullptr, swt_ = nullptr, minv_ = nullptr, mh_ = nullptr,
         mhq_ = nullptr, mhsc_ = nullptr, mhbs_ = nullptr, my_ = nullptr, mhu_ = nullptr;
  // The pair list is sorted in chunks of moe_tpc_ tokens (at most 512 pairs): counters [chunks][NE]
  int moe_tpc_ = 0;
  int moe_chunks(int T) const { return (T + moe_tpc_ - 1) / moe_tpc_; }
  int slots_ = 0, moe_ne_ = 0, moe_nu_ = 0, moe_e_ = 0, moe_f_ = 0;

  void moe_alloc(int NE, int NU, int E, int F) {
    if (moe_ne_ == NE && moe_nu_ == NU && moe_e_ == E && moe_f_ == F) return;
    if (moe_ne_) throw std::runtime_error("moe_alloc: one expert geometry per engine");
    if (NE <= 0 || NE > 512 || NU <= 0 || NU > 64 || NU > NE || E % 256 || F % 256)
      throw std::runtime_error("moe_alloc: unsupported expert geometry");
    moe_ne_ = NE; moe_nu_ = NU; moe_e_ = E; moe_f_ = F;
    slots_ = max_chunk * NU;
    const size_t S = (size_t)slots_;
    mids_ = buf(S * 4); mwts_ = buf(S * 4); sgate_ = buf((size_t)max_chunk * 4);
    moe_tpc_ = std::max(4, (512 / NU) & ~3);  // (a multiple of the 4 tokens of a routing work-group)
    if (moe_tpc_ * NU > 512) throw std::runtime_error("moe_alloc: more than 128 experts per token");
    const size_t nchunks = (size_t)moe_chunks(max_chunk);
    mcount_ = buf(nchunks * NE * 4); moffs_ = buf((size_t)NE * 4); mcursor_ = buf((size_t)NE * 4);
    mtiles_ = buf((1 + 3 * (S + NE)) * 4); mtstart_ = buf((size_t)(NE + 1) * 4);
    stok_ = buf(S * 4); swt_ = buf(S * 4); minv_ = buf(S * 4);
    mh_ = buf(S * F * 4); mhq_ = buf(S * F); mhsc_ = buf(S * (F / 32) * 4); mhbs_ = buf(S * (F / 16) * 2); my_ = buf(S * E * 4);
    if (moe_pre_) mhu_ = buf(S * (F / 32) * 4 + 1024);  // (sa * S of the experts' inputs, act_usum over mhsc_ / mhbs_)
    const uint32_t zero = 0;
    CL_CHECK(clEnqueueFillBuffer(cl_.queue, mcount_, &zero, 4, 0, nchunks * NE * 4, 0, nullptr, nullptr));
  }

  // NE matrices of N rows x K values -> NE matrices of Np rows x Kp values, the added rows and the added blocks of a
  // row zero bytes (every type decodes them to zeros).  K != Kp: the 32-value-block types only (make_weight).
  static std::vector<uint8_t> pad_expert_tensor(uint32_t type, const uint8_t* src, int NE, int N, int K, int Np, int Kp) {
    const bool blk32 = type == GGML_Q8_0 || type == GGML_Q4_0 || type == GGML_IQ4_NL || type == GGML_MXFP4;
    if (K != Kp && (!blk32 || K % 32)) throw std::runtime_error("make_moe_layer: rows of " + std::to_string(K) + " values of this type cannot be padded");
    const size_t bb = arcz_gguf_bytes(type, 1, 256) / 8;  // (bytes of 32 values; used for the block types only)
    const size_t rb = K != Kp ? (size_t)(K / 32) * bb : arcz_gguf_bytes(type, 1, K);
    const size_t prb = K != Kp ? (size_t)(Kp / 32) * bb : rb;
    std::vector<uint8_t> out((size_t)NE * Np * prb, 0);
    for (int e = 0; e < NE; ++e)
      for (int n = 0; n < N; ++n) memcpy(&out[((size_t)e * Np + n) * prb], src + ((size_t)e * N + n) * rb, rb);
    return out;
  }
  // The three expert tensors of a layer: gate and up [NE][F][E], down [NE][E][F], each of its own type.  E and F that are
  // not whole superblocks (the reference's Gemma 4 layers with F = 704, MXFP4 layers of 2880 x 2880) are padded to them,
  // rows and columns, with zeros, as the reference's loader pads (zero/engine_load.h:371-387): the layer then has the
  // rounded-up E and F -- the activations and the residual rows it works on are that wide, their tails zero -- and the
  // added rows of gate and up give h = silu(0) * 0 = 0 for the added columns of down.
  MoeLayer make_moe_layer(const uint32_t type_in[3], const uint8_t* const data[3], int NE, int NU, int E, int F) {
    if (NE <= 0 || E <= 0 || F <= 0) throw std::runtime_error("make_moe_layer: bad shape");
    const int Ep = (E + 255) / 256 * 256, Fp = (F + 255) / 256 * 256;
    std::vector<uint8_t> pad[3], as40[3];
    uint32_t type[3] = {type_in[0], type_in[1], type_in[2]};
    const uint8_t* d[3] = {data[0], data[1], data[2]};
    for (int i = 0; i < 3; ++i) {  // (AR4_128, Q2_0: as Q4_0 blocks first, see as_q4_0)
      const size_t rows = (size_t)NE * (i == 2 ? E : F);
      const int K = i == 2 ? F : E;
      size_t nb = arcz_relayout_q4_0(type[i], rows, K, nullptr, nullptr);
      if (type[i] == GGML_AR4_128 || type[i] == GGML_Q2_0) as_q4_0(type[i], d[i], nb, rows, K, as40[i]);
    }
    if (Ep != E || Fp != F) {
      pad[0] = pad_expert_tensor(type[0], d[0], NE, F, E, Fp, Ep);
      pad[1] = pad_expert_tensor(type[1], d[1], NE, F, E, Fp, Ep);
      pad[2] = pad_expert_tensor(type[2], d[2], NE, E, F, Ep, Fp);
      for (int i = 0; i < 3; ++i) d[i] = pad[i].data();
    }
    moe_alloc(NE, NU, Ep, Fp);
    MoeLayer L;
    L.NE = NE; L.NU = NU; L.E = Ep; L.F = Fp;
    L.ex[0] = make_weight(type[0], d[0], arcz_gguf_bytes(type[0], (size_t)NE * Fp, Ep), Fp, Ep, (size_t)NE * Fp);
    L.ex[1] = make_weight(type[1], d[1], arcz_gguf_bytes(type[1], (size_t)NE * Fp, Ep), Fp, Ep, (size_t)NE * Fp);
    L.ex[2] = make_weight(type[2], d[2], arcz_gguf_bytes(type[2], (size_t)NE * Ep, Fp), Ep, Fp, (size_t)NE * Ep);
    if (moe_pre_ && mhu_)
      for (int i = 0; i < 3; ++i) {
        if (L.ex[i].type != GGML_Q4_K) continue;
        const size_t rows = L.ex[i].rows;
        const int K = L.ex[i].K, nsb = K / 256;
        if (rows * (size_t)(K / 32) >= (1ull << 30)) continue;  // (the kernels form these offsets in 32 bits)
        // (+ 4096: the last expert's last tile reads whole 128-row pieces)
        L.wsv[i] = buf(rows * (size_t)(K / 32) * 8 + 4096);
        cl_kernel kw = kernel("ops", "", "q4k_wscales");
        size_t hdr = planes_q4k(rows, nsb).hdr;
        int NN = (int)rows, nsb2 = nsb;
        set_args(kw, 0, L.ex[i].raw, hdr, NN, nsb2, L.wsv[i]);
        size_t g2[2] = {(rows + 255) / 256 * 256, (size_t)nsb}, l2[2] = {256, 1};
        run("q4k_wscales", kw, 2, g2, l2);
      }
    return L;
  }
  void free_moe_layer(MoeLayer& L) {
    for (int i = 0; i < 3; ++i) {
      free_weight(L.ex[i]);
      if (L.wsv[i]) release(L.wsv[i]);
      L.wsv[i] = nullptr;
    }
    set_moe_routing(L, nullptr, nullptr, 1.0f);
  }
  MoeLayer make_moe_layer(uint32_t type, const uint8_t* gate, const uint8_t* up, const uint8_t* down, int NE, int NU,
                          int E, int F) {
    const uint32_t types[3] = {type, type, type};
    const uint8_t* const data[3] = {gate, up, down};
    return make_moe_layer(types, data, NE, NU, E, F);
  }

  // routing -> slots grouped by expert -> tiles (zero/engine_moe.h:95-134).  rl: router logits [T][ldl] f32.
  // tm: slots per tile.
  // usum (plain routing only): the routing launch also writes au_ = sa * S of the current chunk's rows of K values.
  void moe_route(const MoeLayer& L, cl_mem rl, int ldl, int T, int tm, bool usum = false) {
    const int NE = L.NE, NU = L.NU, n = T * NU;
    if (T <= 0 || T > max_chunk || ldl < NE || arcz_mem_size(rl) < ((size_t)(T - 1) * ldl + NE) * 4)
      throw std::runtime_error("moe_route: router logits do not fit");
    const std::string defs = "-DNE=" + std::to_string(NE) + " -DNU=" + std::to_string(NU) + " -DTM=" + std::to_string(tm) +
                             " -DNPART=" + std::to_string(moe_tpc_) + " -DNCH=" + std::to_string(moe_chunks(T));
    {
      if (usum && L.variant()) throw std::logic_error("moe_route: the routing variants do not write the sums");
      cl_kernel k = kernel("moe", defs + (usum ? " -DUSUM=1" : L.route_defs()), "moe_route");
      int NR = ldl, TT = T;
      set_args(k, 0, rl, NR, TT, mids_, mwts_, sgate_, mcount_);
      if (L.escale) set_args(k, 7, L.escale);  // (zero/engine_moe.h:114-115)
      if (L.ebias) set_args(k, 7, L.ebias);
      if (usum) {
        int MM = cur_Mp_, nblk = cur_K_ / 32;
        set_args(k, 7, asc_, absum_, MM, au_, nblk);
      }
      size_t g1 = (size_t)(T + 3) / 4 * 256, l1 = 256;
      run("moe_route", k, 1, &g1, &l1);
    }
    {
      cl_kernel k = kernel("moe", defs, "moe_scan");
      set_args(k, 0, mcount_, moffs_, mcursor_, mtiles_, mtstart_);
      size_t g1 = 1024, l1 = 1024;
      run("moe_scan", k, 1, &g1, &l1);
    }
    {
      cl_kernel k = kernel("moe", defs, "moe_scatter");
      int nn = n;
      set_args(k, 0, mids_, mwts_, nn, mcount_, stok_, swt_, minv_);  // (the cursor: the chunks' first slots per expert)
      size_t g1 = (size_t)moe_chunks(T) * 512, l1 = 512;
      run("moe_scatter", k, 1, &g1, &l1);
    }
  }

  // The experts of a chunk through the tile GEMM (zero/engine_moe.h:433-470 moe_gemm, without its decode pass: the
  // kernel decodes the raw rows itself): part 0 = gate, then up with the fused SwiGLU into mh_; part 2 = down,
  // routing-weighted, into my_.
  void moe_gemm(const MoeLayer& L, int part, int Mp, size_t max_tiles, int n_slots = 0) {
    const int E = L.E, F = L.F, NE = L.NE;
    for (int i = part; i < (part == 0 ? 2 : 3); ++i) {
      const int N = i == 2 ? E : F, K = i == 2 ? F : E;
      const GpuWeight wx = gemm_form(i == 2 ? "moe_down" : "moe_gateup", L.ex[i]);
      const bool pre = i == 2 && L.wsv[2] && n_slots != 0;
      cl_kernel k = pre ? kernel("gemm", "-DQTYPE=12 -DACT32 -DMOE_TILES -DPRE=1 -DNE=" + std::to_string(NE), "gemm")
                        : gemm_kernel(wx.type, true, NE, wx.half_d);
      int M = i == 2 ? slots_ : Mp, NN = N, KK = K, ldc = N, acc = i == 1 ? 2 : 0, e0 = 0, e1 = NE, um = i == 2 ? 0 : 1,
          us = i == 2 ? 1 : 0;
      cl_mem unused = nullptr;
      if (pre && n_slots > 0) {  // sa * S of the n_slots expert inputs (n_slots < 0: the gate / up kernel wrote them)
        cl_kernel ku = kernel("ops", "", "act_usum");
        set_args(ku, 0, mhsc_, mhbs_, M, mhu_);
        size_t g2[2] = {(size_t)(n_slots + 255) / 256 * 256, (size_t)(K / 32)}, l2[2] = {256, 1};
        run("act_usum", ku, 2, g2, l2);
      }
      set_args(k, 0, wx.raw, unused, i == 2 ? mhq_ : aq_, i == 2 ? mhsc_ : asc_, i == 2 ? mhbs_ : absum_, i == 2 ? my_ : mh_, M, NN, KK,
               ldc, acc, mtiles_, mtstart_, e0, e1, stok_, um, swt_, us);
      if (pre) set_args(k, 19, mhu_, L.wsv[2]);
      // (tile work-groups in a multiple of 8: the kernels deal tiles to the XCDs in runs of the expert-sorted list)
      size_t gws[2] = {(size_t)(N + 127) / 128 * 256, (max_tiles + 7) / 8 * 8}, lws[2] = {256, 1};
      run(i == 2 ? "moe_down" : "moe_gateup", k, 2, gws, lws);
    }
  }

  // x[t] += sum_k w_k * expert_k(h[t]) for the T tokens whose quantized h is the current activation chunk
  // (zero/engine_moe.h:8-361 layer_moe: standard experts, no shared expert).  x: [T][E] f32.
  // sh (may be null): the shared expert's output rows [T][E] f32, added as sgate[t] * sh[t] (zero/kernels/moe.cl:344-352;
  // sgate = sigmoid of the router row's logit past the experts', column NE of a row of ldl > NE values).
  void layer_moe(const MoeLayer& L, cl_mem rl, int ldl, cl_mem x, int T, int Mp, cl_mem sh = nullptr) {
    const int E = L.E, F = L.F, NU = L.NU, n = T * NU;
    if (sh && arcz_mem_size(sh) < (size_t)T * E * 4) throw std::runtime_error("layer_moe: sh is too small");
    if (cur_T_ != T || cur_K_ != E || cur_Mp_ != Mp) throw std::runtime_error("layer_moe: the activations are not this chunk's");
    if (!cur_act32_) throw std::runtime_error("layer_moe: the expert kernels take per-32 activation scales (as the reference's, zero/kernels/gemm.cl:140-142)");
    if (arcz_mem_size(x) < (size_t)T * E * 4) throw std::runtime_error("layer_moe: x is too small");
    // A pass of 1-16 tokens (zero/engine_moe.h:86-262 has this form for 1-8): small tiles through the matrix-vector
    // kernels moe_gateup_q / moe_down_q, routed by one launch (moe_route1 for one token, whose NU experts are the tiles;
    // moe_route_small for more) instead of the 64-slot tile GEMMs, which for one token walked K alone in 8 x 6
    // work-groups (128 us a layer at 128 experts x 768 x 2048; ARCZ_MOE_DECODE=0 brings that back).  At 128 x 8 experts
    // the two forms meet at 24 tokens (170 us); 16 tokens take 112 against 137 us (ARCZ_MOE_DECODE_MAX moves the limit).
    // (the switches of this function are read when the engine is made: a test sets them before it makes its engine)
    const bool dec_off = moe_dec_off_;
    const int dec_max = moe_dec_max_;
    if (!dec_off && T <= dec_max && T * NU <= 512) {
      const int NE = L.NE;
      // (one-slot tiles at every count: eight tokens' 64 pairs hit about 50 experts, so a tile of 8 slots holds 1.3 on
      //  average, and the one-slot kernels are the light ones: 71 us a layer against 113 with 8-slot tiles, 45 against
      //  60 for four tokens; ARCZ_MOE_TMD=2|4|8 sets larger tiles)
      const int tmd_env = moe_tmd_;
      const int tmd = T > 1 && (tmd_env == 2 || tmd_env == 4 || tmd_env == 8) ? tmd_env : 1;
      size_t tiles_max;
      const bool fuse_off = moe_fuse_off_;
      // one or two tokens, everything fused: the gate/up kernel routes the tokens itself (no routing launch: 2 launches
      // a layer; the kernel takes up to 8 tokens, but every work-group routes all of them, and from 4 tokens on the
      // routing launch is the cheaper way: 36.6 against 35.7 us at 4, 65.5 against 56.4 at 8)
      const bool froute = T <= 2 && tmd == 1 && !fuse_off && F % 32 == 0 && NE <= 512 && NU <= 64 && !L.variant();
      if (froute) {
        if (ldl < NE || arcz_mem_size(rl) < ((size_t)(T - 1) * ldl + NE) * 4) throw std::runtime_error("layer_moe: router logits do not fit");
        tiles_max = (size_t)n;
      } else if (T == 1) {
        if (ldl < NE || arcz_mem_size(rl) < (size_t)NE * 4) throw std::runtime_error("layer_moe: router logits do not fit");
        cl_kernel k = kernel("moe", "-DNE=" + std::to_string(NE) + " -DNU=" + std::to_string(NU) + " -DHAS_GATE=" +
                                        std::to_string(ldl > NE ? 1 : 0) + L.route_defs(), "moe_route1");
        set_args(k, 0, rl, sgate_, mtiles_, stok_, swt_, minv_);
        if (L.escale) set_args(k, 6, L.escale);  // (zero/engine_moe.h:103-104)
        if (L.ebias) set_args(k, 6, L.ebias);
        size_t g1 = 64, l1 = 64;
        run("moe_route", k, 1, &g1, &l1);
        tiles_max = (size_t)NU;
      } else if (n <= 512 && NE <= 512 && !L.variant()) {
        // routing, scan and scatter of the few pairs in one work-group (the three launches took 19 us)
        if (ldl < NE || arcz_mem_size(rl) < ((size_t)(T - 1) * ldl + NE) * 4) throw std::runtime_error("layer_moe: router logits do not fit");
        cl_kernel k = kernel("moe", "-DNE=" + std::to_string(NE) + " -DNU=" + std::to_string(NU) + " -DTM=" + std::to_string(tmd),
                             "moe_route_small");
        int NR = ldl, TT = T;
        set_args(k, 0, rl, NR, TT, mids_, mwts_, sgate_, mtiles_, stok_, swt_, minv_);
        size_t g1 = 512, l1 = 512;
        run("moe_route", k, 1, &g1, &l1);
        tiles_max = (size_t)(n + tmd - 1) / tmd + std::min(n, NE);
      } else {
        moe_route(L, rl, ldl, T, tmd);
        tiles_max = (size_t)(n + tmd - 1) / tmd + std::min(n, NE);
      }
      cl_mem tabs = tabs_;
      const std::string dd = " -DGROWS=2 -DTM=" + std::to_string(tmd) + " -DNE=" + std::to_string(NE);
      if (L.ex[0].type != L.ex[1].type) throw std::runtime_error("layer_moe: gate and up experts of different types");
      // Tiles of one or two slots: the gate/up kernel quantizes its own output (32 rows a work-group: one block per
      // slot); one-slot tiles: the down kernel sums a token's experts into x itself.  3 launches instead of 5
      // (ARCZ_MOE_FUSE=0: the 5).
      const bool fq = !fuse_off && tmd <= 2 && F % 32 == 0, fc = !fuse_off && tmd == 1 && NU <= 64 && !sh;
      if (froute) {
        cl_kernel k = kernel("decode", "-DQT=" + std::to_string(L.ex[0].type) + " -DGROWS=4 -DTM=1 -DQUANT=1 -DROUTE=1 -DNE=" +
                                           std::to_string(NE), "moe_gateup_q");
        int FF = F, KK = E, MM = Mp, S = slots_, NUU = NU, NR = ldl, TT = T;
        set_args(k, 0, L.ex[0].raw, L.ex[1].raw, FF, KK, tabs, aq_, asc_, MM, mtiles_, stok_, mh_, absum_, S, mhq_, mhsc_,
                 mhbs_, rl, sgate_, swt_, minv_, NUU, NR, TT, mids_, mwts_);
        size_t gws[2] = {(size_t)(F / 32) * 512, tiles_max}, lws[2] = {512, 1};
        run("moe_gateup", k, 2, gws, lws);
      } else if (fq) {
        cl_kernel k = kernel("decode", "-DQT=" + std::to_string(L.ex[0].type) + " -DGROWS=4 -DTM=" + std::to_string(tmd) +
                                           " -DQUANT=1 -DNE=" + std::to_string(NE), "moe_gateup_q");
        int FF = F, KK = E, MM = Mp, S = slots_;
        set_args(k, 0, L.ex[0].raw, L.ex[1].raw, FF, KK, tabs, aq_, asc_, MM, mtiles_, stok_, mh_, absum_, S, mhq_, mhsc_,
                 mhbs_);
        size_t gws[2] = {(size_t)(F / 32) * 512, tiles_max}, lws[2] = {512, 1};
        run("moe_gateup", k, 2, gws, lws);
      } else {
        {
          cl_kernel k = kernel("decode", "-DQT=" + std::to_string(L.ex[0].type) + dd, "moe_gateup_q");
          int FF = F, KK = E, MM = Mp;
          set_args(k, 0, L.ex[0].raw, L.ex[1].raw, FF, KK, tabs, aq_, asc_, MM, mtiles_, stok_, mh_, absum_);
          size_t gws[2] = {((size_t)(F + 1) / 2 * 32 + 255) / 256 * 256, tiles_max}, lws[2] = {256, 1};
          run("moe_gateup", k, 2, gws, lws);
        }
        {
          cl_kernel k = kernel("moe", "-DNE=" + std::to_string(NE) + " -DNU=" + std::to_string(NU), "moe_quant_sums");
          int FF = F, S = slots_;
          set_args(k, 0, mh_, FF, S, mhq_, mhsc_, mhbs_);
          size_t gws[2] = {(size_t)256 * (F / 256), (size_t)(n + 63) / 64}, lws[2] = {256, 1};
          run("moe_quant", k, 2, gws, lws);
        }
      }
      if (fc) {
        cl_kernel k = kernel("decode", "-DQT=" + std::to_string(L.ex[2].type) + " -DGROWS=4 -DNE=" + std::to_string(NE),
                             "moe_down1_q");
        int NN = E, KK = F, S = slots_;
        int NUU = NU;
        set_args(k, 0, L.ex[2].raw, NN, KK, tabs, mhq_, mhsc_, S, mtiles_, swt_, x, mhbs_, minv_, NUU);
        size_t gws[2] = {((size_t)E + 3) / 4 * 256, (size_t)T}, lws[2] = {256, 1};
        run("moe_down", k, 2, gws, lws);
      } else {
        {
          cl_kernel k = kernel("decode", "-DQT=" + std::to_string(L.ex[2].type) + dd, "moe_down_q");
          int NN = E, KK = F, S = slots_;
          set_args(k, 0, L.ex[2].raw, NN, KK, tabs, mhq_, mhsc_, S, mtiles_, swt_, my_, mhbs_);
          size_t gws[2] = {((size_t)(E + 1) / 2 * 32 + 255) / 256 * 256, tiles_max}, lws[2] = {256, 1};
          run("moe_down", k, 2, gws, lws);
        }
        {
          cl_kernel k = kernel("moe", "-DNE=" + std::to_string(NE) + " -DNU=" + std::to_string(NU), "moe_combine");
          int EE = E;
          set_args(k, 0, x, sh, sgate_, my_, minv_, EE);
          size_t gws[2] = {((size_t)E + 1023) / 1024 * 256, (size_t)T}, lws[2] = {256, 1};
          run("moe_combine", k, 2, gws, lws);
        }
      }
      return;
    }
    // slots per tile = the token rows of one work-group of the tile GEMM: 64 when any of the three tensors is Q4_K,
    // Q5_K or Q6_K (IQ3_S runs as Q6_K) -- their tile kernels take at most 64; the others' take up to 128 and run
    // 64-slot tiles as well -- else 128
    bool t64 = false;
    for (int i = 0; i < 3; ++i)
      t64 = t64 || L.ex[i].type == GGML_Q4_K || L.ex[i].type == GGML_Q5_K || L.ex[i].type == GGML_Q6_K || L.ex[i].type == GGML_IQ3_S ||
            L.ex[i].type == GGML_Q3_K || L.ex[i].type == GGML_IQ3_XXS;
    const int tm = t64 ? 64 : 128;
    // (the ready-made scale vectors: gate and up Q4_K with the quantizing epilogue; the token side's sa * S then comes
    //  from the routing launch, or from a launch of its own with the routing variants)
    const bool pre_gu = L.ex[0].type == GGML_Q4_K && L.ex[1].type == GGML_Q4_K && F % 128 == 0 && !moe_qfuse_off_ &&
                        L.wsv[0] && L.wsv[1];
    moe_route(L, rl, ldl, T, tm, pre_gu && !L.variant());
    // the tile count is only known on the GPU: launch for the most tiles possible (zero/engine_moe.h:153)
    const size_t max_tiles = (size_t)(n + tm - 1) / tm + std::min(n, L.NE);
    bool quant_fused = false;
    if (L.ex[0].type == GGML_Q4_K && L.ex[1].type == GGML_Q4_K) {
      // gate and up in one pass (the reference's moe_gateup_q, zero/kernels/decode_moe.cl:92-94, launched by
      // zero/engine_moe.h:300-330): h = silu(gate) * up into mh_
      // ... and, when F is whole tiles of 128 rows, the expert inputs' quantization in the same kernel's epilogue
      // (-DQUANT=1: hq / hsc / hbs as moe_quant_sums makes them, bit for bit; ARCZ_MOE_QFUSE=0: the separate launch)
      quant_fused = F % 128 == 0 && !moe_qfuse_off_;
      const bool pre = pre_gu;
      cl_kernel k = kernel("gemm", std::string(pre ? "-DQT=12 -DQUANT=1 -DPRE=2 -DNE=" : quant_fused ? "-DQT=12 -DQUANT=1 -DNE=" : "-DQT=12 -DNE=") + std::to_string(L.NE), "moe_gateup_q");
      int FF = F, KK = E, MM = Mp, S = slots_;
      cl_mem tabs = nullptr;
      if (pre && L.variant()) {  // sa * S of the chunk's tokens
        cl_kernel ku = kernel("ops", "", "act_usum");
        set_args(ku, 0, asc_, absum_, MM, au_);
        size_t g2[2] = {(size_t)(Mp + 255) / 256 * 256, (size_t)(E / 32)}, l2[2] = {256, 1};
        run("act_usum", ku, 2, g2, l2);
      }
      if (pre)
        set_args(k, 0, L.ex[0].raw, L.ex[1].raw, FF, KK, tabs, aq_, asc_, MM, mtiles_, stok_, mh_, absum_, S, mhq_, mhsc_, mhbs_,
                 au_, L.wsv[0], L.wsv[1], L.wsv[2] ? mhu_ : nullptr);
      else if (quant_fused)
        set_args(k, 0, L.ex[0].raw, L.ex[1].raw, FF, KK, tabs, aq_, asc_, MM, mtiles_, stok_, mh_, absum_, S, mhq_, mhsc_, mhbs_);
      else
        set_args(k, 0, L.ex[0].raw, L.ex[1].raw, FF, KK, tabs, aq_, asc_, MM, mtiles_, stok_, mh_, absum_);
      size_t gws[2] = {(size_t)(F + 127) / 128 * 256, (max_tiles + 7) / 8 * 8}, lws[2] = {256, 1};  // (a multiple of 8: moe_tile_of)
      run("moe_gateup", k, 2, gws, lws);
    } else {
      moe_gemm(L, 0, Mp, max_tiles);
    }
    if (!quant_fused) {
      // (the reference's moe_quant writes no sums; the Q4_K tile GEMM here takes them for its min term)
      cl_kernel k = kernel("moe", "-DNE=" + std::to_string(L.NE) + " -DNU=" + std::to_string(NU), "moe_quant_sums");
      int FF = F, S = slots_;
      set_args(k, 0, mh_, FF, S, mhq_, mhsc_, mhbs_);
      size_t gws[2] = {(size_t)256 * (F / 256), (size_t)(n + 63) / 64}, lws[2] = {256, 1};
      run("moe_quant", k, 2, gws, lws);
    }
    moe_gemm(L, 2, Mp, max_tiles, pre_gu ? -1 : n);  // (-1: mhu_ is written already)
    {
      cl_kernel k = kernel("moe", "-DNE=" + std::to_string(L.NE) + " -DNU=" + std::to_string(NU), "moe_combine");
      int EE = E;
      set_args(k, 0, x, sh, sgate_, my_, minv_, EE);
      size_t gws[2] = {((size_t)E + 1023) / 1024 * 256, (size_t)T}, lws[2] = {256, 1};  // (four columns a thread)
      run("moe_combine", k, 2, gws, lws);
    }
  }

 private:
  void check_chunk(int K, int Mp, int T) {
    if (K <= 0 || K % 256 || K > max_k || Mp <= 0 || Mp > max_chunk || T <= 0 || T > Mp)
      throw std::runtime_error("activation chunk " + std::to_string(T) + " of " + std::to_string(Mp) + " rows x " +
                               std::to_string(K) + " does not fit the engine's buffers (" + std::to_string(max_chunk) + " x " +
                               std::to_string(max_k) + ")");
  }
  std::map<std::string, cl_kernel> kernels_;
  std::vector<cl_program> progs_;
  std::vector<cl_mem> mems_;
  std::vector<std::pair<std::string, cl_event>> events_;
};
// Start-up check in the pattern of the reference's xmx_check (zero/engine_setup.h:424-520): every tuned GEMM the
// dispatch can take -- for each weight type, storing, accumulating and with the fused SwiGLU epilogue, in one piece
// and with K shared out over several work-groups per tile -- against the plain kernel of the same type on the
// reference's LCG data, with unit scales (weights d = 1, sub-scales 1, Q4_K / Q5_K mins 1; activation scales 1) so that
// every f32 sum is an integer below 2^24: the two results must be bit-equal to each other and, for store and add, to
// the integer sums counted on the host.  Returns an empty string, or what differed.
inline std::string engine_self_check() {
  const int M = 128, N = 128;
  uint32_t lcg = 12345u;
  auto next = [&]() { lcg = lcg * 1664525u + 1013904223u; return lcg >> 8; };
  static const int iq4[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};
  // one superblock with unit scales and random quants; wq: the integer each element stands for
  auto make_sb = [&](uint32_t type, uint8_t* blk, int* wq) {
    if (type == GGML_Q8_0) {
      for (int b = 0; b < 8; ++b) {
        uint8_t* p = blk + 34 * b;
        p[0] = 0x00; p[1] = 0x3C;  // f16 1.0
        for (int i = 0; i < 32; ++i) {
          const int q = (int)(next() % 255u) - 127;
          p[2 + i] = (uint8_t)(int8_t)q;
          wq[b * 32 + i] = q;
        }
      }
    } else if (type == GGML_Q4_0 || type == GGML_IQ4_NL || type == GGML_MXFP4) {
      static const int fp4[16] = {0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12};
      const int hb = type == GGML_MXFP4 ? 1 : 2;  // bytes of a block's scale: E8M0 128 = 2^0, or f16 1.0
      for (int b = 0; b < 8; ++b) {
        uint8_t* p = blk + (16 + hb) * b;
        if (hb == 1) { p[0] = 128; } else { p[0] = 0x00; p[1] = 0x3C; }
        for (int i = 0; i < 16; ++i) {
          const int lo = (int)(next() & 15u), hi = (int)(next() & 15u);
          p[hb + i] = (uint8_t)(lo | hi << 4);
          wq[b * 32 + i] = type == GGML_Q4_0 ? lo - 8 : type == GGML_IQ4_NL ? iq4[lo] : fp4[lo];
          wq[b * 32 + 16 + i] = type == GGML_Q4_0 ? hi - 8 : type == GGML_IQ4_NL ? iq4[hi] : fp4[hi];
        }
      }
    } else if (type == GGML_Q4_K || type == GGML_Q5_K) {
      const bool q5 = type == GGML_Q5_K;
      memset(blk, 0, q5 ? 176 : 144);
      blk[0] = 0x00; blk[1] = 0x3C; blk[2] = 0x00; blk[3] = 0x3C;  // d = dmin = 1.0
      for (int i = 0; i < 8; ++i) blk[4 + i] = 1;                   // 6-bit scales and mins of sub-blocks 0-3: 1
      for (int i = 0; i < 4; ++i) blk[12 + i] = 0x11;               // low nibbles of those of sub-blocks 4-7: 1
      uint8_t *qh = blk + 16, *qs = blk + (q5 ? 48 : 16);
      for (int j = 0; j < 4; ++j)
        for (int l = 0; l < 32; ++l) {
          const int lim = q5 ? 31 : 15;
          const int lo = (int)(next() & lim), hi = (int)(next() & lim);
          qs[j * 32 + l] = (uint8_t)((lo & 15) | (hi & 15) << 4);
          if (q5) qh[l] |= (uint8_t)(((lo >> 4) << (2 * j)) | ((hi >> 4) << (2 * j + 1)));
          wq[j * 64 + l] = lo - 1;  // value = 1 * 1 * q - 1 * 1
          wq[j * 64 + 32 + l] = hi - 1;
        }
    } else if (type == GGML_Q6_K) {
      memset(blk, 0, 210);
      for (int i = 0; i < 16; ++i) blk[192 + i] = 1;  // int8 scales
      blk[208] = 0x00; blk[209] = 0x3C;
      for (int n2 = 0; n2 < 2; ++n2)
        for (int l = 0; l < 32; ++l) {
          int q[4];
          for (int k = 0; k < 4; ++k) { q[k] = (int)(next() & 63u); wq[128 * n2 + 32 * k + l] = q[k] - 32; }
          blk[64 * n2 + l] = (uint8_t)((q[0] & 15) | (q[2] & 15) << 4);
          blk[64 * n2 + 32 + l] = (uint8_t)((q[1] & 15) | (q[3] & 15) << 4);
          blk[128 + 32 * n2 + l] = (uint8_t)((q[0] >> 4) | (q[1] >> 4) << 2 | (q[2] >> 4) << 4 | (q[3] >> 4) << 6);
        }
    } else {  // IQ4_XS: 6-bit scales 33 (- 32 = 1): low nibble 1, high two bits 2
      memset(blk, 0, 136);
      blk[0] = 0x00; blk[1] = 0x3C; blk[2] = 0xAA; blk[3] = 0xAA;
      for (int i = 0; i < 4; ++i) blk[4 + i] = 0x11;
      for (int b = 0; b < 8; ++b)
        for (int j = 0; j < 16; ++j) {
          const int lo = (int)(next() & 15u), hi = (int)(next() & 15u);
          blk[8 + 16 * b + j] = (uint8_t)(lo | hi << 4);
          wq[32 * b + j] = iq4[lo];
          wq[32 * b + 16 + j] = iq4[hi];
        }
    }
  };
  // K = 1024: one piece (few superblocks); K = 2048 with smaller activations: the tile's K in four pieces
  for (int K : {1024, 2048}) {
    Engine e(M, K);
    const int amax = K == 1024 ? 127 : 63;
    std::vector<int8_t> aq((size_t)M * K);
    std::vector<float> asc((size_t)M * (K / 32), 1.0f);
    std::vector<int16_t> absum((size_t)M * (K / 16));
    for (auto& v : aq) v = (int8_t)((int)(next() % (unsigned)(2 * amax + 1)) - amax);
    for (int m = 0; m < M; ++m)
      for (int b = 0; b < K / 16; ++b) {
        int sm = 0;
        for (int i = 0; i < 16; ++i) sm += aq[(size_t)m * K + b * 16 + i];
        absum[(size_t)b * M + m] = (int16_t)sm;
      }
    e.set_activations(aq.data(), asc.data(), absum.data(), K, M, M);
    cl_mem c0 = e.buf((size_t)M * N * 4), c1 = e.buf((size_t)M * N * 4);
    std::vector<float> y0((size_t)M * N), y1((size_t)M * N), cinit((size_t)M * N);
    for (auto& v : cinit) v = (float)((int)(next() % 9u) - 4);  // small integers: sums with them stay exact
    for (uint32_t type : {GGML_Q8_0, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K, GGML_IQ4_XS, GGML_Q4_0, GGML_IQ4_NL, GGML_MXFP4}) {
      const size_t rb = arcz_gguf_bytes(type, 1, K), sbb = rb / (size_t)(K / 256);
      std::vector<uint8_t> w((size_t)N * rb);
      std::vector<int> wq((size_t)N * K);
      for (int n = 0; n < N; ++n)
        for (int sb = 0; sb < K / 256; ++sb) make_sb(type, &w[n * rb + sb * sbb], &wq[(size_t)n * K + sb * 256]);
      GpuWeight gw = e.make_weight(type, w.data(), w.size(), N, K);
      for (int mode = 0; mode < 3; ++mode) {
        CL_CHECK(clEnqueueWriteBuffer(e.cl_.queue, c0, CL_TRUE, 0, cinit.size() * 4, cinit.data(), 0, nullptr, nullptr));
        CL_CHECK(clEnqueueWriteBuffer(e.cl_.queue, c1, CL_TRUE, 0, cinit.size() * 4, cinit.data(), 0, nullptr, nullptr));
        e.gemm_dense("self_check", gw, M, c0, N, 0, mode);  // the kernel(s) the engine's dispatch takes for this type
        {
          cl_kernel k = e.kernel("gemm", "-DQTYPE=" + std::to_string(type) + " -DACT32", "gemm_simple");
          cl_mem unused = nullptr;
          int MM = M, NN = N, KK = K, ldc = N, zero = 0, one = 1, s1 = K / 256, md = mode;
          set_args(k, 0, gw.raw, unused, e.aq_, e.asc_, e.absum_, c1, MM, NN, KK, ldc, zero, md, one, zero, s1);
          size_t gws[1] = {(size_t)(M / 128) * (N / 128) * 256}, lws[1] = {256};
          e.run("self_check", k, 1, gws, lws);
        }
        CL_CHECK(clEnqueueReadBuffer(e.cl_.queue, c0, CL_TRUE, 0, y0.size() * 4, y0.data(), 0, nullptr, nullptr));
        CL_CHECK(clEnqueueReadBuffer(e.cl_.queue, c1, CL_TRUE, 0, y1.size() * 4, y1.data(), 0, nullptr, nullptr));
        for (int m = 0; m < M; ++m)
          for (int n = 0; n < N; ++n) {
            long long sm = 0;
            for (int k2 = 0; k2 < K; ++k2) sm += (long long)aq[(size_t)m * K + k2] * wq[(size_t)n * K + k2];
            const float a = y0[(size_t)m * N + n], b = y1[(size_t)m * N + n];
            const float want = mode == 0 ? (float)sm : mode == 1 ? (float)sm + cinit[(size_t)m * N + n] : a;
            uint32_t ab, bb;
            memcpy(&ab, &a, 4);
            memcpy(&bb, &b, 4);
            if (ab != bb || a != want || !std::isfinite(a)) {
              e.free_weight(gw);
              return std::string("GEMM self-check ") + ggml_type_name(type) + " K=" + std::to_string(K) + " mode " +
                     std::to_string(mode) + ": token " + std::to_string(m) + " row " + std::to_string(n) + ": tuned " +
                     std::to_string(a) + ", simple " + std::to_string(b) + ", integer sum " + std::to_string(sm);
            }
          }
      }
      e.free_weight(gw);
    }
  }
  return std::string();
}
