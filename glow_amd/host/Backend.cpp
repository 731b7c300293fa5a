// Compile side of the MI355X backend: verifies each lowered instruction,
// derives the integer kernel parameters the way Glow's CPU code generator does
// (reference lib/LLVMIRCodeGen/LLVMIRGen.cpp:618-662, 1670-1690, 2161-2320,
// 2501-2599, 2695-2798, 3638-3659) and emits a list of C-ABI launches.
#include "Backend.h"

#include "glow_mi355x.h"

#include <algorithm>
#include <cmath>
#include <sstream>

namespace glow_mi355x {

namespace {

struct S32To8 { int32_t pre, post, scale; };
S32To8 s32to8(float ratio) {
  int32_t o[4];
  mi355x_quantize_scale_offset_32to8(ratio, 0, o);
  return {o[0], o[1], o[2]};
}

// Requantisation hint of a launch whose per-column parameters are these host
// vectors (bias values from the constant's payload; boffs NULL = boff for all).
int requantHintFor(size_t K, int32_t inOff, int32_t outOff, const int32_t *wOffs, const void *bias,
                   int bias8, const int32_t *boffs, int32_t boff, const std::vector<int32_t> &bpre,
                   const std::vector<int32_t> &bpost, const std::vector<int32_t> &bscale,
                   const std::vector<int32_t> &opre, const std::vector<int32_t> &opost,
                   const std::vector<int32_t> &oscale) {
  int flags = 0;
  if (mi355x_gemm_requant_hint_host(K, opre.size(), inOff, outOff, wOffs, bias, bias8, boffs, boff,
                                    bpre.data(), bpost.data(), bscale.data(), opre.data(),
                                    opost.data(), oscale.data(), &flags) != MI355X_OK)
    return 0;
  return flags;
}

bool shiftsOk(const S32To8 &p) { return p.pre >= 0 && p.pre <= 31 && p.post >= 0 && p.post <= 31; }

// quantization::quantize<int32_t> (reference Base.h:323-329)
int32_t quantizeI32(float x, float scale, int32_t offset) {
  float r = x / scale + (float)offset;
  double v = std::nearbyintf(r);
  if (v > 2147483647.0) v = 2147483647.0;
  if (v < -2147483648.0) v = -2147483648.0;
  return (int32_t)v;
}

// Byte offsets of compiler-made buffers inside the generated region.
class Generated {
public:
  // initialised int32 vector
  size_t addI32(const std::vector<int32_t> &v) {
    const size_t off = image_.size();
    image_.resize(alignUp(off + v.size() * 4, kTensorAlignment), 0);
    std::memcpy(image_.data() + off, v.data(), v.size() * 4);
    return off;
  }
  size_t addBytes(const std::vector<int8_t> &v) {
    const size_t off = image_.size();
    image_.resize(alignUp(off + v.size(), kTensorAlignment), 0);
    std::memcpy(image_.data() + off, v.data(), v.size());
    return off;
  }
  // uninitialised scratch placed after every initialised buffer
  size_t addScratch(size_t bytes) {
    const size_t off = scratch_;
    scratch_ = alignUp(scratch_ + bytes, 256);
    return off; // relative to scratchBase(), fixed up by the caller at the end
  }
  std::vector<uint8_t> image_;
  size_t scratch_ = 0;
};

struct Operand {
  const Value *v;
  // an activation's place in its region, in the compiled function's table
  // (filled when every launch of the function is known)
  const size_t *actOffset = nullptr;
  // region + offset -> device pointer at launch time
  uint8_t *ptr(const DeviceBindings &b) const {
    switch (v->category) {
    case SymbolCategory::Constant: return b.constants + v->offset;
    case SymbolCategory::Placeholder: return b.mutableMem + v->offset;
    default: return b.activations + (actOffset ? *actOffset : v->offset);
    }
  }
  const Type &ty() const { return v->type; }
};

std::string kv(const char *k, long long v) { return strFormat(" %s=%lld", k, v); }

std::string vecStr(const char *k, const std::vector<int32_t> &v) {
  std::string s = strFormat(" %s=[", k);
  for (size_t i = 0; i < v.size(); i++) s += (i ? "," : "") + std::to_string(v[i]);
  return s + "]";
}

} // namespace

#define CHECK_OP(cond, ...)                                                    \
  do {                                                                         \
    if (!(cond))                                                               \
      return MI355X_MAKE_ERR(ErrorCode::COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE, \
                             "%s '%s': %s", kindName(I.kind), I.name.c_str(),  \
                             strFormat(__VA_ARGS__).c_str());                  \
  } while (0)

namespace {

class Compiler {
public:
  // `function` is the index of the function whose activations may be used;
  // a negative one accepts any activation (single-instruction probes).
  Compiler(const Module &M, const std::vector<Instruction> &insts, int function,
           const BackendOptions &o)
      : M_(M), insts_(insts), function_(function), opts_(o),
        actOff_(std::make_shared<std::vector<size_t>>((size_t)M.numValues(), 0)) {
    for (int id = 0; id < M.numValues(); id++) (*actOff_)[(size_t)id] = M.value(id).offset;
  }

  Error run(MI355XFunction &out) {
    for (const auto &I : insts_) MI355X_RETURN_IF_ERR(checkOperands(I));
    absorbed_.assign(insts_.size(), 0);
    for (size_t at = 0; at < insts_.size(); at++) {
      if (absorbed_[at]) continue; // folded into an earlier launch
      const Instruction &I = insts_[at];
      const size_t firstLaunch = out.launches.size(), firstInst = at;
      std::vector<size_t> folded;   // instructions further down that this launch also covers
      switch (I.kind) {
      case Kind::ElementAdd: {
        // an add whose only reader is the Relu right behind it becomes one pass
        const Instruction *relu = nullptr;
        if (opts_.fuseAddRelu && at + 1 < insts_.size() && insts_[at + 1].kind == Kind::Relu &&
            insts_[at + 1].operands[1] == I.operands[0] &&
            M_.value(I.operands[0]).category == SymbolCategory::Activation &&
            readers(I.operands[0]) == 1)
          relu = &insts_[at + 1];
        MI355X_RETURN_IF_ERR(add(I, relu, out));
        if (relu) at++;
        break;
      }
      case Kind::Relu: MI355X_RETURN_IF_ERR(relu(I, out)); break;
      case Kind::Clip:
      case Kind::LeakyRelu:
      case Kind::CPUMaxSplat: MI355X_RETURN_IF_ERR(elementUnary(I, out)); break;
      case Kind::BatchedAdd: MI355X_RETURN_IF_ERR(batchedAdd(I, out)); break;
      case Kind::MaxPool: MI355X_RETURN_IF_ERR(pool(I, out, false)); break;
      case Kind::AvgPool: MI355X_RETURN_IF_ERR(pool(I, out, true)); break;
      case Kind::SoftMax: MI355X_RETURN_IF_ERR(softmax(I, out)); break;
      case Kind::RowwiseQuantizedSparseLengthsWeightedSum:
      case Kind::EmbeddingBagByteRowwiseOffsets: MI355X_RETURN_IF_ERR(otherLookups(I, out)); break;
      case Kind::Transpose: {
        // a {0,2,1} shuffle read only by the BatchMatMul right behind it as its
        // right operand: the product reads the untransposed tensor instead
        if (opts_.fuseTransposeMatMul && at + 1 < insts_.size() &&
            insts_[at + 1].kind == Kind::BatchMatMul &&
            insts_[at + 1].operands[2] == I.operands[0] &&
            insts_[at + 1].operands[1] != I.operands[0] &&
            I.iattrs == std::vector<int64_t>{0, 2, 1} &&
            M_.value(I.operands[0]).category == SymbolCategory::Activation &&
            readers(I.operands[0]) == 1 && matmulNtOk(I, insts_[at + 1])) {
          // ... and a Gather of single elements of the product (then maybe the
          // InsertTensor of what it gathers) behind it
          std::vector<int32_t> destOf;
          const size_t g = opts_.fuseInsert ? soleGatherOf(at + 1, destOf) : 0;
          const size_t ins = g ? soleInsertOf(at + 1, insts_[g].operands[0], insts_[at + 1]) : 0;
          MI355X_RETURN_IF_ERR(matmulNt(I, insts_[at + 1], out, g ? &insts_[g] : nullptr, destOf,
                                        ins ? &insts_[ins] : nullptr));
          if (g) { absorbed_[g] = 1; folded.push_back(g); }
          if (ins) { absorbed_[ins] = 1; folded.push_back(ins); }
          at++;
        } else {
          MI355X_RETURN_IF_ERR(movement(I, out));
        }
        break;
      }
      case Kind::ConvertTo:
      case Kind::InsertTensor:
      case Kind::BatchMatMul:
      case Kind::Copy:
      case Kind::Sigmoid: MI355X_RETURN_IF_ERR(movement(I, out)); break;
      case Kind::Gather: {
        // a result that is only inserted into a wider tensor is gathered there
        const size_t ins =
            opts_.fuseInsert && I.iattrs.size() == 1 && I.iattrs[0] == 1 ? soleInsertOf(at) : 0;
        MI355X_RETURN_IF_ERR(movement(I, out, ins ? &insts_[ins] : nullptr));
        if (ins) { absorbed_[ins] = 1; folded.push_back(ins); }
        break;
      }
      case Kind::Quantize: {
        // a Quantize read only by the convolution right behind it: when that
        // convolution goes through space-to-depth (the stem of an image
        // network), the layout change quantizes on the way
        const Instruction *cv = at + 1 < insts_.size() ? &insts_[at + 1] : nullptr;
        const bool convKind = cv && (cv->kind == Kind::Convolution ||
                                     cv->kind == Kind::ChannelwiseQuantizedConvolution);
        if (opts_.fuseQuantizeStem && convKind && cv->operands[1] == I.operands[0] &&
            M_.value(I.operands[0]).category == SymbolCategory::Activation &&
            M_.value(I.operands[0]).type.kind == ElemKind::Int8QTy &&
            M_.value(I.operands[0]).type.dims.size() == 4 && readers(I.operands[0]) == 1 &&
            writers(I.operands[0]) == 1 &&
            !(at + 2 < insts_.size() && insts_[at + 2].kind == Kind::ElementAdd)) {
          MI355X_RETURN_IF_ERR(conv(*cv, out, cv->kind == Kind::ChannelwiseQuantizedConvolution,
                                    nullptr, nullptr, &I));
          at++;
        } else {
          MI355X_RETURN_IF_ERR(quantize(I, out));
        }
        break;
      }
      case Kind::Dequantize: {
        // a Sigmoid right behind it that is the only reader of its result
        const Instruction *sig = nullptr;
        if (opts_.fuseDequantizeSigmoid && at + 1 < insts_.size() &&
            insts_[at + 1].kind == Kind::Sigmoid && insts_[at + 1].operands[1] == I.operands[0] &&
            M_.value(I.operands[0]).category == SymbolCategory::Activation &&
            readers(I.operands[0]) == 1 &&
            M_.value(insts_[at + 1].operands[0]).type.kind == ElemKind::FloatTy &&
            M_.value(insts_[at + 1].operands[0]).type.size() == M_.value(I.operands[0]).type.size())
          sig = &insts_[at + 1];
        // ... or a SoftMax over its rows
        const Instruction *smax = nullptr;
        if (!sig && opts_.fuseDequantizeSigmoid && at + 1 < insts_.size() &&
            insts_[at + 1].kind == Kind::SoftMax && insts_[at + 1].operands[1] == I.operands[0] &&
            M_.value(I.operands[0]).category == SymbolCategory::Activation &&
            readers(I.operands[0]) == 1 && writers(I.operands[0]) == 1 &&
            M_.value(I.operands[1]).type.kind == ElemKind::Int8QTy &&
            M_.value(I.operands[0]).type.dims.size() == 2 &&
            M_.value(insts_[at + 1].operands[0]).type.kind == ElemKind::FloatTy &&
            M_.value(insts_[at + 1].operands[0]).type.dims == M_.value(I.operands[0]).type.dims &&
            M_.value(I.operands[1]).type.size() == M_.value(I.operands[0]).type.size())
          smax = &insts_[at + 1];
        MI355X_RETURN_IF_ERR(dequantize(I, out, sig, smax));
        if (sig || smax) at++;
        break;
      }
      case Kind::RescaleQuantized: {
        const size_t ins = opts_.fuseInsert ? soleInsertOf(at) : 0;
        MI355X_RETURN_IF_ERR(rescale(I, out, ins ? &insts_[ins] : nullptr));
        if (ins) { absorbed_[ins] = 1; folded.push_back(ins); }
        break;
      }
      case Kind::FullyConnected: MI355X_RETURN_IF_ERR(fc(I, out)); break;
      case Kind::RowwiseQuantizedFullyConnected: {
        // a Relu instruction right behind it that is the only reader of its result
        const Instruction *reluI = nullptr;
        if (opts_.fuseFcRelu && at + 1 < insts_.size() && insts_[at + 1].kind == Kind::Relu &&
            insts_[at + 1].operands[1] == I.operands[0] &&
            M_.value(I.operands[0]).category == SymbolCategory::Activation &&
            readers(I.operands[0]) == 1 &&
            M_.value(insts_[at + 1].operands[0]).type.kind == ElemKind::Int8QTy &&
            M_.value(insts_[at + 1].operands[0]).type.dims == M_.value(I.operands[0]).type.dims)
          reluI = &insts_[at + 1];
        MI355X_RETURN_IF_ERR(rwqfc(I, out, reluI));
        if (reluI) at++;
        break;
      }
      case Kind::MatMul: MI355X_RETURN_IF_ERR(matmul(I, out)); break;
      case Kind::Convolution: MI355X_RETURN_IF_ERR(conv(I, out, false)); break;
      case Kind::ChannelwiseQuantizedConvolution: {
        if (M_.value(I.operands[1]).type.dims.size() == 5) {   // NTHWC: the 3-D form
          MI355X_RETURN_IF_ERR(conv3d(I, out));
          break;
        }
        // conv -> ElementAdd(conv, residual) [-> Relu] with no other reader of
        // the intermediate tensors: one kernel
        const Instruction *addI = nullptr, *reluI = nullptr;
        if (opts_.fuseConvAdd && at + 1 < insts_.size() && insts_[at + 1].kind == Kind::ElementAdd) {
          const Instruction &A = insts_[at + 1];
          const int cd = I.operands[0];
          const bool lhs = A.operands[1] == cd, rhs = A.operands[2] == cd;
          if ((lhs != rhs) && M_.value(cd).category == SymbolCategory::Activation &&
              readers(cd) == 1 && M_.value(cd).type.dims == M_.value(A.operands[0]).type.dims) {
            addI = &A;
            if (opts_.fuseAddRelu && at + 2 < insts_.size() && insts_[at + 2].kind == Kind::Relu &&
                insts_[at + 2].operands[1] == A.operands[0] &&
                M_.value(A.operands[0]).category == SymbolCategory::Activation &&
                readers(A.operands[0]) == 1)
              reluI = &insts_[at + 2];
          }
        }
        MI355X_RETURN_IF_ERR(conv(I, out, true, addI, reluI));
        at += (addI ? 1 : 0) + (reluI ? 1 : 0);
        break;
      }
      case Kind::FusedRowwiseQuantizedSparseLengthsWeightedSum:
        MI355X_RETURN_IF_ERR(slws(I, out, true)); break;
      case Kind::FusedRowwiseQuantizedSparseLengthsSum: {
        const size_t used = opts_.fuseSlsChains ? multiSls(at, out) : 0;
        if (used) at += used - 1;
        else MI355X_RETURN_IF_ERR(slws(I, out, false));
        break;
      }
      default:
        return MI355X_MAKE_ERR(ErrorCode::COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE,
                               "instruction kind %d is not supported", (int)I.kind);
      }
      // what the launches of instructions [firstInst, at] read and write
      for (size_t l = firstLaunch; l < out.launches.size(); l++) {
        for (size_t k = firstInst; k <= at; k++) noteAccesses(insts_[k], out.launches[l]);
        for (size_t k : folded) noteAccesses(insts_[k], out.launches[l]);
        const std::string &kn = out.launches[l].kernel;
        out.launches[l].tunable = kn == "mi355x_fc_i8" || kn == "mi355x_rwq_fc_i8" ||
                                  kn == "mi355x_matmul_i8" || kn == "mi355x_conv2d_i8" ||
                                  kn == "mi355x_cwq_conv2d_i8" || kn == "mi355x_cwq_conv2d_add_i8" ||
                                  kn == "mi355x_rwq_fc_relu_i8";
      }
    }
    planActivations(out);
    assignLevels(out);
    // scratch buffers follow the initialised image
    scratchBase_ = alignUp(gen_.image_.size(), 256);
    *scratchBasePtr_ = scratchBase_;
    out.generated = std::move(gen_.image_);
    genTotal_ = scratchBase_ + gen_.scratch_;
    return Error::success();
  }

  size_t generatedTotal() const { return genTotal_; }
  const std::map<int, std::pair<bool, bool>> &io() const { return io_; }

private:
  static constexpr int kArity[(int)Kind::NumKinds] = {2, 2, 2, 4, 6, 3, 4, 8, 5, 4, 3, 2, 2, 2, 2,
                                                       2, 2, 2, 3, 3, 2, 7, 5, 2, 2, 2, 2, 3};

  Error checkOperands(const Instruction &I) {
    CHECK_OP((int)I.kind >= 0 && (int)I.kind < (int)Kind::NumKinds, "unknown kind");
    CHECK_OP((int)I.operands.size() == kArity[(int)I.kind], "expects %d operands, has %zu",
             kArity[(int)I.kind], I.operands.size());
    for (size_t i = 0; i < I.operands.size(); i++) {
      const int id = I.operands[i];
      CHECK_OP(M_.validId(id), "operand %zu is not a value of the module", i);
      const Value &v = M_.value(id);
      CHECK_OP(v.category != SymbolCategory::Activation || function_ < 0 ||
                   v.function == function_,
               "operand %zu is an activation of another function", i);
      CHECK_OP(!(i == 0 && v.category == SymbolCategory::Constant),
               "destination is a constant");
      // (a placeholder read or written through a view is an input or output itself)
      for (int who : {id, v.root}) {
        auto &f = io_[who];
        if (i == 0) f.second = true; else f.first = true;
      }
    }
    return Error::success();
  }

  Operand op(const Instruction &I, int i) const { return opOf(M_.value(I.operands[(size_t)i])); }
  Operand opOf(const Value &v) const { return Operand{&v, &(*actOff_)[(size_t)v.id]}; }

  void noteAccesses(const Instruction &J, KernelLaunch &L) const {
    // (Pooled lookups over more than 4096 bags use scratch inside the kernel
    // library that belongs to the stream they are launched on, so launches on
    // different branches of the graph need no ordering for its sake.)
    for (size_t i = 0; i < J.operands.size(); i++) {
      const Value &v = M_.value(J.operands[i]);
      Access a;
      a.root = v.root;
      if (J.kind == Kind::InsertTensor && i == 0 && v.type.dims.size() == 2) {
        // only the columns [offset, offset + width) of each row are written
        const Value &src = M_.value(J.operands[1]);
        const long long es = (long long)elemSize(v.type.kind);
        a.lo = J.iattrs.empty() ? 0 : J.iattrs[0] * es;
        a.hi = a.lo + (src.type.dims.size() == 2 ? src.type.dims[1] * es : 0);
        if (v.id != v.root) a.hi = -1; // a view's rows need not line up with its source's
      }
      (i == 0 ? L.writes : L.reads).push_back(a);
    }
  }

  // Places the function's activations (AllocationsInfo::allocateActivations,
  // AllocationsInfo.cpp:128-156, over MemoryAllocator::allocate,
  // MemoryAllocator.cpp:58-91: first fit by address). Launches, not
  // instructions, are the unit of a value's life, because a fused launch reads
  // and writes all of its instructions' operands at once; and a life ends not
  // at a position in the launch list but in the dependence graph (see deadFor),
  // because the launches of independent chains run side by side. Values no
  // launch touches get no memory. The byte ranges are recorded in the accesses,
  // so that `conflict` sees launches whose values share bytes.
  void planActivations(MI355XFunction &out) {
    auto &L = out.launches;
    const size_t nv = (size_t)M_.numValues();
    std::vector<long long> first(nv, -1), last(nv, -1);
    auto isAct = [&](int root) {
      return root >= 0 && M_.value(root).category == SymbolCategory::Activation;
    };
    for (size_t i = 0; i < L.size(); i++)
      for (const auto *set : {&L[i].reads, &L[i].writes})
        for (const Access &a : *set)
          if (isAct(a.root)) {
            if (first[(size_t)a.root] < 0) first[(size_t)a.root] = (long long)i;
            last[(size_t)a.root] = (long long)i;
          }
    constexpr size_t kAlign = 256;
    std::vector<size_t> rootOff(nv, 0), rootSize(nv, 0);
    size_t total = 0;
    auto bytesOf = [&](size_t r) {
      return alignUp(std::max<size_t>(1, M_.value((int)r).type.sizeInBytes()), kAlign);
    };
    // A value that a single launch both writes and reads, and no other launch
    // touches, is a result handed from one instruction to the next inside a
    // fused launch: the kernel keeps it in registers. It gets no memory of its
    // own (it is put at the start of the region, which is at least its size).
    std::vector<char> inner(nv, 0);
    if (opts_.reuseActivations)
      for (size_t r = 0; r < nv; r++) {
        if (first[r] < 0 || first[r] != last[r]) continue;
        const KernelLaunch &l = L[(size_t)first[r]];
        bool rd = false, wr = false;
        for (const Access &a : l.reads) rd = rd || a.root == (int)r;
        for (const Access &a : l.writes) wr = wr || a.root == (int)r;
        if (rd && wr) {
          inner[r] = 1;
          rootSize[r] = bytesOf(r);
          total = std::max(total, rootSize[r]);
          first[r] = last[r] = -1;
        }
      }
    if (opts_.reuseActivations) {
      // anc[i]: the launches that run before launch i in every order the
      // dependences allow (its ancestors in the graph of conflicts by value)
      const size_t n = L.size(), words = (n + 63) / 64;
      std::vector<std::vector<uint64_t>> anc(n, std::vector<uint64_t>(words, 0));
      for (size_t i = 0; i < n; i++)
        for (size_t j = i; j-- > 0;) {
          if ((anc[i][j / 64] >> (j % 64)) & 1) continue;
          if (!conflict(L[j], L[i])) continue;
          anc[i][j / 64] |= 1ull << (j % 64);
          for (size_t w = 0; w < words; w++) anc[i][w] |= anc[j][w];
        }
      std::vector<std::vector<size_t>> touchers(nv);
      for (size_t i = 0; i < n; i++)
        for (const auto *set : {&L[i].reads, &L[i].writes})
          for (const Access &a : *set)
            if (isAct(a.root) && first[(size_t)a.root] >= 0 &&
                (touchers[(size_t)a.root].empty() || touchers[(size_t)a.root].back() != i))
              touchers[(size_t)a.root].push_back(i);
      // The bytes of value q may pass to value r when every launch that touches
      // q is an ancestor of every launch that touches r (r may have several
      // independent writers, e.g. slices inserted by parallel chains): the
      // hand-over then adds no ordering that the data flow does not already
      // impose, so independent chains stay independent.
      auto deadFor = [&](int q, size_t r) {
        for (size_t tr : touchers[r])
          for (size_t tq : touchers[(size_t)q])
            if (!((anc[tr][tq / 64] >> (tq % 64)) & 1)) return false;
        return true;
      };
      struct Seg { size_t lo, hi; int root; };
      std::vector<Seg> segs;                    // disjoint, sorted by address
      for (size_t i = 0; i < n; i++)
        for (size_t r = 0; r < nv; r++) {
          if (first[r] != (long long)i) continue;
          const size_t need = bytesOf(r);
          // first fit: the lowest address whose bytes are free or dead for r
          size_t at = 0;
          for (bool moved = true; moved;) {
            moved = false;
            for (const Seg &g : segs)
              if (g.lo < at + need && at < g.hi && !deadFor(g.root, r)) {
                at = g.hi;
                moved = true;
              }
          }
          // what r covers of the dead values' segments is taken from them
          std::vector<Seg> next;
          for (const Seg &g : segs) {
            if (g.hi <= at || g.lo >= at + need) { next.push_back(g); continue; }
            if (g.lo < at) next.push_back(Seg{g.lo, at, g.root});
            if (g.hi > at + need) next.push_back(Seg{at + need, g.hi, g.root});
          }
          next.push_back(Seg{at, at + need, (int)r});
          std::sort(next.begin(), next.end(), [](const Seg &x, const Seg &y) { return x.lo < y.lo; });
          segs.swap(next);
          rootOff[r] = at;
          rootSize[r] = need;
          total = std::max(total, at + need);
        }
    } else {
      for (size_t r = 0; r < nv; r++) {
        if (first[r] < 0) continue;
        rootSize[r] = bytesOf(r);
        rootOff[r] = total;
        total += rootSize[r];
      }
    }
    // views lie where their root lies
    for (size_t id = 0; id < nv; id++) {
      const Value &v = M_.value((int)id);
      if (v.category != SymbolCategory::Activation) continue;
      if (function_ >= 0 && v.function != function_) continue;
      (*actOff_)[id] = isAct(v.root) ? rootOff[(size_t)v.root] : 0;
    }
    for (auto &l : L)
      for (auto *set : {&l.reads, &l.writes})
        for (Access &a : *set)
          if (isAct(a.root) && !inner[(size_t)a.root]) {
            a.actLo = (long long)rootOff[(size_t)a.root];
            a.actHi = a.actLo + (long long)rootSize[(size_t)a.root];
          }
    for (size_t r = 0; r < nv; r++)
      if (first[r] >= 0)
        out.activationPlan.push_back({M_.value((int)r).name, (int)r, rootOff[r], rootSize[r]});
    out.activationOffsets = actOff_;
    out.activationsBytes = total;
  }

  static bool conflict(const KernelLaunch &early, const KernelLaunch &late) {
    for (const auto &w : early.writes) {
      for (const auto &r : late.reads) if (w.overlaps(r)) return true;   // read after write
      for (const auto &x : late.writes) if (w.overlaps(x)) return true;  // write after write
    }
    for (const auto &r : early.reads)
      for (const auto &w : late.writes) if (r.overlaps(w)) return true;  // write after read
    return false;
  }

  // level = longest chain of conflicting launches in front of a launch
  static void assignLevels(MI355XFunction &out) {
    auto &L = out.launches;
    for (size_t i = 0; i < L.size(); i++) {
      int lvl = 0;
      for (size_t j = 0; j < i; j++)
        if (L[j].level >= lvl && conflict(L[j], L[i])) lvl = L[j].level + 1;
      L[i].level = lvl;
    }
  }

  // number of operands that read the memory of `id` (through it or a view)
  int readers(int id) const {
    const int root = M_.value(id).root;
    int n = 0;
    for (const auto &I : insts_)
      for (size_t i = 1; i < I.operands.size(); i++)
        n += M_.validId(I.operands[i]) && M_.value(I.operands[i]).root == root;
    return n;
  }

  int writers(int id) const {
    const int root = M_.value(id).root;
    int n = 0;
    for (const auto &I : insts_)
      n += M_.validId(I.operands[0]) && M_.value(I.operands[0]).root == root;
    return n;
  }

  // The InsertTensor (its position, 0 if none) that is the only reader of the
  // 2-D result of instruction `at` and can take effect at `at` already: nothing
  // in between reads the tensor it inserts into, and whatever writes that
  // tensor in between is an InsertTensor of other columns.
  size_t soleInsertOf(size_t at) const { return soleInsertOf(at, insts_[at].operands[0], insts_[at]); }

  // The same for value `v`, which launch `P` at position `at` is going to write
  // (P's own result, or that of an instruction folded into P).
  size_t soleInsertOf(size_t at, int v, const Instruction &P) const {
    const Value &pv = M_.value(v);
    if (pv.category != SymbolCategory::Activation || pv.root != v || pv.type.dims.size() != 2 ||
        readers(v) != 1 || writers(v) != 1)
      return 0;
    size_t j = at + 1;
    for (; j < insts_.size(); j++) {
      bool reads = false;
      for (size_t i = 1; i < insts_[j].operands.size(); i++) reads = reads || insts_[j].operands[i] == v;
      if (reads) break;
    }
    if (j >= insts_.size()) return 0;
    const Instruction &J = insts_[j];
    if (J.kind != Kind::InsertTensor || J.operands[1] != v || J.iattrs.size() != 1 || J.iattrs[0] < 0)
      return 0;
    const Value &D = M_.value(J.operands[0]);
    if (D.type.dims.size() != 2 || D.type.kind != pv.type.kind || D.type.dims[0] != pv.type.dims[0] ||
        J.iattrs[0] + pv.type.dims[1] > D.type.dims[1] || D.root == pv.root)
      return 0;
    if (isQuantized(D.type.kind) && (D.type.scale != pv.type.scale || D.type.offset != pv.type.offset))
      return 0;
    // the producer itself must not read the tensor it would now write
    for (size_t i = 1; i < P.operands.size(); i++)
      if (M_.value(P.operands[i]).root == D.root) return 0;
    const int64_t lo = J.iattrs[0], hi = lo + pv.type.dims[1];
    for (size_t k = at + 1; k < j; k++) {
      const Instruction &K = insts_[k];
      for (size_t i = 1; i < K.operands.size(); i++)
        if (M_.value(K.operands[i]).root == D.root) return 0;
      if (M_.value(K.operands[0]).root != D.root) continue;
      if (K.kind != Kind::InsertTensor || K.operands[0] != J.operands[0] || K.iattrs.size() != 1)
        return 0;
      const int64_t klo = K.iattrs[0], khi = klo + M_.value(K.operands[1]).type.dims.back();
      if (klo < hi && lo < khi) return 0;
    }
    return j;
  }

  // where a producer folded with InsertTensor `ins` writes: the wide tensor,
  // the byte offset of the slice in a row, and the row pitch in bytes
  struct SliceDest {
    Operand wide;
    size_t offset, pitch;
  };
  SliceDest sliceDest(const Instruction &ins) const {
    Operand wide = op(ins, 0);
    const size_t es = elemSize(wide.ty().kind);
    return {wide, (size_t)ins.iattrs[0] * es, (size_t)wide.ty().dims[1] * es};
  }

  Error add(const Instruction &I, const Instruction *reluI, MI355XFunction &out) {
    Operand d = op(I, 0), l = op(I, 1), r = op(I, 2);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && l.ty().kind == ElemKind::Int8QTy &&
                 r.ty().kind == ElemKind::Int8QTy,
             "needs i8 operands");
    CHECK_OP(d.ty().size() == l.ty().size() && d.ty().size() == r.ty().size(), "size mismatch");
    const size_t n = (size_t)d.ty().size();
    const S32To8 lp = s32to8(l.ty().scale / d.ty().scale), rp = s32to8(r.ty().scale / d.ty().scale);
    const int32_t doff = d.ty().offset, lo = l.ty().offset, ro = r.ty().offset;
    std::string params = strFormat(" n=%zu", n) + kv("dest_offset", doff) + kv("lhs_offset", lo) +
                         kv("rhs_offset", ro) + kv("lhs_pre", lp.pre) + kv("lhs_post", lp.post) +
                         kv("lhs_scale", lp.scale) + kv("rhs_pre", rp.pre) + kv("rhs_post", rp.post) +
                         kv("rhs_scale", rp.scale);
    if (!reluI) {
      out.launches.push_back({"mi355x_add_i8", I.name, params, [=](const DeviceBindings &b) {
                                return mi355x_add_i8((int8_t *)d.ptr(b), (const int8_t *)l.ptr(b),
                                                     (const int8_t *)r.ptr(b), n, doff, lo, ro, lp.pre,
                                                     lp.post, lp.scale, rp.pre, rp.post, rp.scale,
                                                     b.stream);
                              }});
      return Error::success();
    }
    const Instruction &R = *reluI;
    Operand rd = op(R, 0);
    {
      const Instruction &I = R; // for the message
      CHECK_OP(rd.ty().kind == ElemKind::Int8QTy && rd.ty().size() == d.ty().size(),
               "needs an i8 result of the same size");
    }
    const S32To8 dp = s32to8(d.ty().scale / rd.ty().scale);
    const int32_t rdo = rd.ty().offset;
    params += kv("relu_dest_offset", rdo) + kv("relu_pre", dp.pre) + kv("relu_post", dp.post) +
              kv("relu_scale", dp.scale);
    out.launches.push_back({"mi355x_add_relu_i8", I.name + "+" + R.name, params,
                            [=](const DeviceBindings &b) {
                              return mi355x_add_relu_i8((int8_t *)rd.ptr(b), (const int8_t *)l.ptr(b),
                                                        (const int8_t *)r.ptr(b), n, doff, lo, ro,
                                                        lp.pre, lp.post, lp.scale, rp.pre, rp.post,
                                                        rp.scale, rdo, dp.pre, dp.post, dp.scale,
                                                        b.stream);
                            }});
    return Error::success();
  }

  Error relu(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), s = op(I, 1);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && s.ty().kind == ElemKind::Int8QTy, "needs i8 -> i8");
    CHECK_OP(d.ty().size() == s.ty().size(), "size mismatch");
    const size_t n = (size_t)d.ty().size();
    const S32To8 p = s32to8(s.ty().scale / d.ty().scale);
    const int32_t so = s.ty().offset, doff = d.ty().offset;
    out.launches.push_back(
        {"mi355x_relu_i8", I.name,
         strFormat(" n=%zu", n) + kv("src_offset", so) + kv("dest_offset", doff) + kv("pre", p.pre) +
             kv("post", p.post) + kv("scale", p.scale),
         [=](const DeviceBindings &b) {
           return mi355x_relu_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), n, so, doff, p.pre,
                                 p.post, p.scale, b.stream);
         }});
    return Error::success();
  }

  // ClipInst, LeakyReluInst and CPUMaxSplatInst on int8 (reference
  // LLVMIRGen.cpp:1501-1590, CPULLVMIRGen.cpp:135-167).
  Error elementUnary(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), s = op(I, 1);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && s.ty().kind == ElemKind::Int8QTy, "needs i8 -> i8");
    CHECK_OP(d.ty().size() == s.ty().size(), "size mismatch");
    const size_t n = (size_t)d.ty().size();
    const int32_t so = s.ty().offset, doff = d.ty().offset;
    auto q8 = [&](float x) {
      // quantization::quantize<int8_t> with the source tensor's parameters
      const int32_t v = quantizeI32(x, s.ty().scale, so);
      return v < -128 ? -128 : (v > 127 ? 127 : v);
    };
    if (I.kind == Kind::Clip) {
      CHECK_OP(I.fattrs.size() == 2, "Clip needs {min, max}");
      const int32_t lo = q8(I.fattrs[0]), hi = q8(I.fattrs[1]);
      const S32To8 p = s32to8(s.ty().scale / d.ty().scale);
      out.launches.push_back(
          {"mi355x_clip_i8", I.name,
           strFormat(" n=%zu", n) + kv("clip_min", lo) + kv("clip_max", hi) + kv("src_offset", so) +
               kv("dest_offset", doff) + kv("pre", p.pre) + kv("post", p.post) + kv("scale", p.scale),
           [=](const DeviceBindings &b) {
             return mi355x_clip_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), n, lo, hi, so, doff,
                                   p.pre, p.post, p.scale, b.stream);
           }});
      return Error::success();
    }
    if (I.kind == Kind::LeakyRelu) {
      CHECK_OP(I.fattrs.size() == 1, "LeakyRelu needs {alpha}");
      const S32To8 pp = s32to8(s.ty().scale / d.ty().scale);
      const S32To8 np = s32to8(s.ty().scale * I.fattrs[0] / d.ty().scale);
      out.launches.push_back(
          {"mi355x_leaky_relu_i8", I.name,
           strFormat(" n=%zu", n) + kv("src_offset", so) + kv("dest_offset", doff) +
               kv("pos_pre", pp.pre) + kv("pos_post", pp.post) + kv("pos_scale", pp.scale) +
               kv("neg_pre", np.pre) + kv("neg_post", np.post) + kv("neg_scale", np.scale),
           [=](const DeviceBindings &b) {
             return mi355x_leaky_relu_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), n, so, doff,
                                         pp.pre, pp.post, pp.scale, np.pre, np.post, np.scale,
                                         b.stream);
           }});
      return Error::success();
    }
    // Max(x, Splat(v)) keeps its operand's type (the node the CPU backend makes
    // of it has one)
    CHECK_OP(I.fattrs.size() == 1, "CPUMaxSplat needs {splatValue}");
    CHECK_OP(d.ty().scale == s.ty().scale && doff == so,
             "source and destination must share scale and offset");
    const int32_t v = q8(I.fattrs[0]);
    out.launches.push_back({"mi355x_max_splat_i8", I.name, strFormat(" n=%zu", n) + kv("value", v),
                            [=](const DeviceBindings &b) {
                              return mi355x_max_splat_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b),
                                                         n, v, b.stream);
                            }});
    return Error::success();
  }

  // BatchedAddInst on an int8 batch with an int8 or int32 slice (reference
  // LLVMIRGen.cpp:2322-2375).
  Error batchedAdd(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), bt = op(I, 1), sl = op(I, 2);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && bt.ty().kind == ElemKind::Int8QTy,
             "needs an i8 batch and result");
    CHECK_OP(sl.ty().kind == ElemKind::Int8QTy || sl.ty().kind == ElemKind::Int32QTy,
             "needs an i8 or i32 slice");
    CHECK_OP(d.ty().dims == bt.ty().dims, "batch and result differ in shape");
    CHECK_OP(!bt.ty().dims.empty() && bt.ty().dims[0] > 0 &&
                 sl.ty().size() * bt.ty().dims[0] == bt.ty().size(),
             "slice %s is not one slice of batch %s", sl.ty().str().c_str(), bt.ty().str().c_str());
    const size_t numSlice = (size_t)bt.ty().dims[0], sliceSize = (size_t)sl.ty().size();
    const int i32 = sl.ty().kind == ElemKind::Int32QTy;
    const S32To8 bp = s32to8(bt.ty().scale / d.ty().scale);
    const S32To8 sp = s32to8(sl.ty().scale / d.ty().scale);
    const int32_t doff = d.ty().offset, bo = bt.ty().offset, so = sl.ty().offset;
    out.launches.push_back(
        {"mi355x_batched_add_i8", I.name,
         strFormat(" slices=%zu slice_size=%zu", numSlice, sliceSize) + kv("slice_is_i32", i32) +
             kv("dest_offset", doff) + kv("batch_offset", bo) + kv("slice_offset", so) +
             kv("batch_pre", bp.pre) + kv("batch_post", bp.post) + kv("batch_scale", bp.scale) +
             kv("slice_pre", sp.pre) + kv("slice_post", sp.post) + kv("slice_scale", sp.scale),
         [=](const DeviceBindings &b) {
           return mi355x_batched_add_i8((int8_t *)d.ptr(b), (const int8_t *)bt.ptr(b), sl.ptr(b), i32,
                                        numSlice, sliceSize, doff, bo, so, bp.pre, bp.post, bp.scale,
                                        sp.pre, sp.post, sp.scale, b.stream);
         }});
    return Error::success();
  }

  Error pool(const Instruction &I, MI355XFunction &out, bool avg) {
    Operand d = op(I, 0), s = op(I, 1);
    CHECK_OP((int)I.iattrs.size() == (avg ? 9 : 8), "expects %d integer attributes", avg ? 9 : 8);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && s.ty().kind == ElemKind::Int8QTy, "needs i8 -> i8");
    CHECK_OP(d.ty().dims.size() == 4 && s.ty().dims.size() == 4, "needs NHWC tensors");
    const auto &a = I.iattrs;
    for (int i = 0; i < 8; i++) CHECK_OP(a[(size_t)i] >= 0, "negative attribute");
    CHECK_OP(a[0] > 0 && a[1] > 0 && a[2] > 0 && a[3] > 0, "kernel and stride must be positive");
    const size_t N = (size_t)s.ty().dims[0], IH = (size_t)s.ty().dims[1], IW = (size_t)s.ty().dims[2],
                 C = (size_t)s.ty().dims[3];
    const int64_t oh = ((int64_t)IH + a[4] + a[6] - a[0]) / a[2] + 1;
    const int64_t ow = ((int64_t)IW + a[5] + a[7] - a[1]) / a[3] + 1;
    CHECK_OP(d.ty().dims[0] == (int64_t)N && d.ty().dims[3] == (int64_t)C && d.ty().dims[1] == oh &&
                 d.ty().dims[2] == ow,
             "output %s does not match the computed %lld x %lld", d.ty().str().c_str(), (long long)oh,
             (long long)ow);
    const size_t OH = (size_t)oh, OW = (size_t)ow, kH = (size_t)a[0], kW = (size_t)a[1],
                 sH = (size_t)a[2], sW = (size_t)a[3], pT = (size_t)a[4], pL = (size_t)a[5];
    const int32_t doff = d.ty().offset;
    std::string geom = strFormat(" N=%zu IH=%zu IW=%zu C=%zu OH=%zu OW=%zu KH=%zu KW=%zu sH=%zu sW=%zu "
                                 "padT=%zu padL=%zu",
                                 N, IH, IW, C, OH, OW, kH, kW, sH, sW, pT, pL);
    if (!avg) {
      // the reference passes the values through: both sides share their parameters
      CHECK_OP(d.ty().scale == s.ty().scale && d.ty().offset == s.ty().offset,
               "input and output must share scale and offset");
      out.launches.push_back({"mi355x_max_pool_i8", I.name, geom + kv("out_offset", doff),
                              [=](const DeviceBindings &b) {
                                return mi355x_max_pool_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b),
                                                          N, IH, IW, C, OH, OW, kH, kW, sH, sW, pT, pL,
                                                          doff, b.stream);
                              }});
      return Error::success();
    }
    const int cip = a[8] != 0;
    float sc = s.ty().scale / d.ty().scale;
    if (cip) sc = sc / (float)(a[0] * a[1]);
    const S32To8 p = s32to8(sc);
    const int32_t so = s.ty().offset;
    out.launches.push_back(
        {"mi355x_avg_pool_i8", I.name,
         geom + kv("count_include_pads", cip) + kv("out_offset", doff) + kv("in_offset", so) +
             kv("pre", p.pre) + kv("post", p.post) + kv("scale", p.scale),
         [=](const DeviceBindings &b) {
           return mi355x_avg_pool_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), N, IH, IW, C, OH, OW,
                                     kH, kW, sH, sW, pT, pL, cip, doff, so, p.pre, p.post, p.scale,
                                     b.stream);
         }});
    return Error::success();
  }

  // data movement and the small operators of ranking models
  Error movement(const Instruction &I, MI355XFunction &out, const Instruction *ins = nullptr) {
    Operand d = op(I, 0), s = op(I, 1);
    switch (I.kind) {
    case Kind::ConvertTo: {
      CHECK_OP(d.ty().kind == ElemKind::FloatTy && s.ty().kind == ElemKind::Float16Ty,
               "only float16 -> float is supported");
      CHECK_OP(d.ty().size() == s.ty().size(), "size mismatch");
      const size_t n = (size_t)d.ty().size();
      out.launches.push_back({"mi355x_convert_f16_to_f32", I.name, strFormat(" n=%zu", n),
                              [=](const DeviceBindings &b) {
                                return mi355x_convert_f16_to_f32((float *)d.ptr(b), s.ptr(b), n, b.stream);
                              }});
      return Error::success();
    }
    case Kind::Copy: {
      // libjit_copy_buffer / CopyInst: the bytes of Src into Dest
      CHECK_OP(d.ty().kind == s.ty().kind && d.ty().sizeInBytes() == s.ty().sizeInBytes(),
               "needs two tensors of one element kind and size");
      CHECK_OP(!isQuantized(d.ty().kind) || (d.ty().scale == s.ty().scale && d.ty().offset == s.ty().offset),
               "source and destination must share scale and offset");
      const size_t n = d.ty().sizeInBytes();
      out.launches.push_back({"mi355x_copy_u8", I.name, strFormat(" bytes=%zu", n),
                              [=](const DeviceBindings &b) {
                                return mi355x_copy_u8(d.ptr(b), s.ptr(b), n, b.stream);
                              }});
      return Error::success();
    }
    case Kind::Sigmoid: {
      CHECK_OP(d.ty().kind == ElemKind::FloatTy && s.ty().kind == ElemKind::FloatTy, "needs float tensors");
      CHECK_OP(d.ty().size() == s.ty().size(), "size mismatch");
      const size_t n = (size_t)d.ty().size();
      out.launches.push_back({"mi355x_sigmoid_f32", I.name, strFormat(" n=%zu", n),
                              [=](const DeviceBindings &b) {
                                return mi355x_sigmoid_f32((float *)d.ptr(b), (const float *)s.ptr(b), n, b.stream);
                              }});
      return Error::success();
    }
    case Kind::InsertTensor: {
      CHECK_OP(d.ty().kind == s.ty().kind && d.ty().dims.size() == 2 && s.ty().dims.size() == 2,
               "needs 2-D tensors of one element kind");
      CHECK_OP(!isQuantized(d.ty().kind) || (d.ty().scale == s.ty().scale && d.ty().offset == s.ty().offset),
               "slice and tensor must share scale and offset");
      CHECK_OP(I.iattrs.size() == 1 && I.iattrs[0] >= 0, "expects the inner offset");
      const size_t es = elemSize(d.ty().kind);
      const size_t rows = (size_t)s.ty().dims[0], w = (size_t)s.ty().dims[1], W = (size_t)d.ty().dims[1];
      const size_t off = (size_t)I.iattrs[0];
      CHECK_OP(d.ty().dims[0] == s.ty().dims[0] && off + w <= W, "slice does not fit");
      out.launches.push_back({"mi355x_insert_rows", I.name,
                              strFormat(" rows=%zu row_bytes=%zu stride=%zu offset=%zu", rows, w * es, W * es, off * es),
                              [=](const DeviceBindings &b) {
                                return mi355x_insert_rows(d.ptr(b), s.ptr(b), rows, w * es, W * es, off * es, b.stream);
                              }});
      return Error::success();
    }
    case Kind::Transpose: {
      CHECK_OP(d.ty().kind == s.ty().kind && !isFused(s.ty().kind), "needs tensors of one plain element kind");
      CHECK_OP(!isQuantized(s.ty().kind) || (d.ty().scale == s.ty().scale && d.ty().offset == s.ty().offset),
               "input and output must share scale and offset");
      const auto &sd = s.ty().dims;
      const auto &dd = d.ty().dims;
      size_t batch = 1, rows = 0, cols = 0;
      const bool i8 = s.ty().kind == ElemKind::Int8QTy;
      if (i8 && I.iattrs == std::vector<int64_t>{1, 0} && sd.size() == 2) {
        rows = (size_t)sd[0]; cols = (size_t)sd[1];
        CHECK_OP(dd.size() == 2 && dd[0] == sd[1] && dd[1] == sd[0], "shape mismatch");
      } else if (i8 && I.iattrs == std::vector<int64_t>{0, 2, 1} && sd.size() == 3) {
        batch = (size_t)sd[0]; rows = (size_t)sd[1]; cols = (size_t)sd[2];
        CHECK_OP(dd.size() == 3 && dd[0] == sd[0] && dd[1] == sd[2] && dd[2] == sd[1], "shape mismatch");
      } else {
        // any other shuffle of up to six dimensions, any element size
        const size_t nd = sd.size();
        CHECK_OP(nd >= 1 && nd <= 6 && I.iattrs.size() == nd && dd.size() == nd,
                 "needs a shuffle of 1 to 6 dimensions");
        std::vector<size_t> dims(nd), shuf(nd);
        unsigned seen = 0;
        for (size_t i = 0; i < nd; i++) {
          CHECK_OP(I.iattrs[i] >= 0 && (size_t)I.iattrs[i] < nd && !(seen & (1u << I.iattrs[i])),
                   "the shuffle is not a permutation");
          seen |= 1u << I.iattrs[i];
          dims[i] = (size_t)sd[i];
          shuf[i] = (size_t)I.iattrs[i];
        }
        for (size_t i = 0; i < nd; i++) CHECK_OP(dd[i] == sd[shuf[i]], "shape mismatch");
        const size_t es = elemSize(s.ty().kind);
        std::string sh;
        for (size_t i = 0; i < nd; i++) sh += (i ? "," : "") + std::to_string(shuf[i]);
        out.launches.push_back({"mi355x_transpose_nd", I.name,
                                strFormat(" dims=%zu elem_size=%zu shuffle=[%s]", nd, es, sh.c_str()),
                                [=](const DeviceBindings &b) {
                                  return mi355x_transpose_nd(d.ptr(b), s.ptr(b), dims.data(), shuf.data(),
                                                             nd, es, b.stream);
                                }});
        return Error::success();
      }
      out.launches.push_back({"mi355x_batch_transpose_i8", I.name,
                              strFormat(" batch=%zu rows=%zu cols=%zu", batch, rows, cols),
                              [=](const DeviceBindings &b) {
                                return mi355x_batch_transpose_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b),
                                                                 batch, rows, cols, b.stream);
                              }});
      return Error::success();
    }
    case Kind::Gather: {
      Operand idx = op(I, 2);
      CHECK_OP(d.ty().kind == s.ty().kind, "data and result must have one element kind");
      CHECK_OP(idx.ty().kind == ElemKind::Int64ITy || idx.ty().kind == ElemKind::Int32ITy,
               "indices must be int64 or int32");
      CHECK_OP(idx.ty().dims.size() == 1, "indices must be 1-D");
      CHECK_OP(I.iattrs.size() == 1 && (I.iattrs[0] == 0 || I.iattrs[0] == 1), "batchDims must be 0 or 1");
      const size_t bd = (size_t)I.iattrs[0];
      const auto &sd = s.ty().dims;
      CHECK_OP(sd.size() > bd, "data has too few dimensions");
      size_t slice = elemSize(s.ty().kind);
      for (size_t i = bd + 1; i < sd.size(); i++) slice *= (size_t)sd[i];
      const size_t samples = bd ? (size_t)sd[0] : 1, sample = (size_t)sd[bd] * slice;
      const size_t nIdx = (size_t)idx.ty().size();
      CHECK_OP((size_t)d.ty().sizeInBytes() == samples * nIdx * slice, "result size mismatch");
      const int i64 = idx.ty().kind == ElemKind::Int64ITy;
      if (ins) {
        const SliceDest sl = sliceDest(*ins);
        out.launches.push_back(
            {"mi355x_gather_rows", I.name + "+" + ins->name,
             strFormat(" num_indices=%zu slice_bytes=%zu samples=%zu sample_bytes=%zu stride=%zu offset=%zu",
                       nIdx, slice, samples, sample, sl.pitch, sl.offset),
             [=](const DeviceBindings &b) {
               return mi355x_gather_rows(sl.wide.ptr(b) + sl.offset, s.ptr(b), idx.ptr(b), i64, nIdx, slice,
                                         samples, sample, sl.pitch, b.stream);
             }});
        return Error::success();
      }
      out.launches.push_back({"mi355x_gather", I.name,
                              strFormat(" num_indices=%zu slice_bytes=%zu samples=%zu sample_bytes=%zu", nIdx, slice, samples, sample),
                              [=](const DeviceBindings &b) {
                                return mi355x_gather(d.ptr(b), s.ptr(b), idx.ptr(b), i64, nIdx, slice, samples, sample, b.stream);
                              }});
      return Error::success();
    }
    default: { // BatchMatMul
      Operand r = op(I, 2);
      CHECK_OP(d.ty().kind == ElemKind::Int8QTy && s.ty().kind == ElemKind::Int8QTy &&
                   r.ty().kind == ElemKind::Int8QTy,
               "needs i8 operands");
      CHECK_OP(d.ty().dims.size() == 3 && s.ty().dims.size() == 3 && r.ty().dims.size() == 3,
               "needs 3-D operands");
      const size_t B = (size_t)s.ty().dims[0], M = (size_t)s.ty().dims[1], K = (size_t)s.ty().dims[2],
                   N = (size_t)r.ty().dims[2];
      CHECK_OP((size_t)r.ty().dims[0] == B && (size_t)r.ty().dims[1] == K && (size_t)d.ty().dims[0] == B &&
                   (size_t)d.ty().dims[1] == M && (size_t)d.ty().dims[2] == N,
               "shape mismatch");
      CHECK_OP((M + N) * K <= 64 * 1024, "matrices too large for the small-matrix kernel");
      const S32To8 p = s32to8(s.ty().scale * r.ty().scale / d.ty().scale);
      const int32_t oo = d.ty().offset, lo = s.ty().offset, ro = r.ty().offset;
      out.launches.push_back({"mi355x_batch_matmul_i8", I.name,
                              strFormat(" B=%zu M=%zu K=%zu N=%zu", B, M, K, N) + kv("out_offset", oo) +
                                  kv("lhs_offset", lo) + kv("rhs_offset", ro) + kv("out_pre", p.pre) +
                                  kv("out_post", p.post) + kv("out_scale", p.scale),
                              [=](const DeviceBindings &b) {
                                return mi355x_batch_matmul_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b),
                                                              (const int8_t *)r.ptr(b), B, M, K, N, oo, lo, ro,
                                                              p.pre, p.post, p.scale, b.stream);
                              }});
      return Error::success();
    }
    }
  }

  // Whether Transpose T followed by BatchMatMul B fits the K-contiguous kernel.
  bool matmulNtOk(const Instruction &T, const Instruction &B) const {
    const Type &src = M_.value(T.operands[1]).type, &tr = M_.value(T.operands[0]).type;
    const Type &lhs = M_.value(B.operands[1]).type, &dst = M_.value(B.operands[0]).type;
    if (src.kind != ElemKind::Int8QTy || tr.kind != ElemKind::Int8QTy ||
        lhs.kind != ElemKind::Int8QTy || dst.kind != ElemKind::Int8QTy)
      return false;
    if (src.dims.size() != 3 || tr.dims.size() != 3 || lhs.dims.size() != 3 || dst.dims.size() != 3)
      return false;
    if (src.scale != tr.scale || src.offset != tr.offset) return false;
    // src [B,N,K] -> tr [B,K,N]; lhs [B,M,K]; dst [B,M,N]
    const int64_t Bn = src.dims[0], N = src.dims[1], K = src.dims[2], Mm = lhs.dims[1];
    if (tr.dims[0] != Bn || tr.dims[1] != K || tr.dims[2] != N) return false;
    if (lhs.dims[0] != Bn || lhs.dims[2] != K) return false;
    if (dst.dims[0] != Bn || dst.dims[1] != Mm || dst.dims[2] != N) return false;
    return K % 16 == 0 && Mm < (1 << 15) && N < (1 << 15) &&
           M_.value(T.operands[1]).offset % 16 == 0 && M_.value(B.operands[1]).offset % 16 == 0;
  }

  // The Gather (its position, 0 if none) that is the only reader of the result
  // of the BatchMatMul at `at`, picks single elements of each sample's flattened
  // matrix by a constant list without repeats, and keeps the quantization
  // parameters: the product can then write the picked elements directly.
  // `destOf` receives, per element of a sample's matrix, its place in the
  // gathered row or -1.
  size_t soleGatherOf(size_t at, std::vector<int32_t> &destOf) const {
    const Instruction &P = insts_[at];
    const int z = P.operands[0];
    const Value &zv = M_.value(z);
    if (zv.category != SymbolCategory::Activation || zv.root != z || zv.type.dims.size() != 3 ||
        readers(z) != 1 || writers(z) != 1)
      return 0;
    size_t j = at + 1;
    for (; j < insts_.size(); j++) {
      bool touches = false;
      for (size_t i = 0; i < insts_[j].operands.size(); i++)
        touches = touches || M_.value(insts_[j].operands[i]).root == z;
      if (touches) break;
    }
    if (j >= insts_.size()) return 0;
    const Instruction &G = insts_[j];
    if (G.kind != Kind::Gather || G.iattrs != std::vector<int64_t>{1}) return 0;
    const Value &src = M_.value(G.operands[1]), &idx = M_.value(G.operands[2]),
                &dst = M_.value(G.operands[0]);
    const int64_t per = zv.type.dims[1] * zv.type.dims[2];
    if (src.root != z || src.offset != zv.offset || src.type.dims.size() != 2 ||
        src.type.dims[0] != zv.type.dims[0] || src.type.dims[1] != per ||
        src.type.kind != ElemKind::Int8QTy)
      return 0;
    if (idx.category != SymbolCategory::Constant || idx.type.dims.size() != 1 ||
        (idx.type.kind != ElemKind::Int64ITy && idx.type.kind != ElemKind::Int32ITy))
      return 0;
    if (dst.category != SymbolCategory::Activation || dst.root != G.operands[0] ||
        dst.type.kind != ElemKind::Int8QTy || dst.type.dims.size() != 2 ||
        dst.type.dims[0] != zv.type.dims[0] || dst.type.dims[1] != idx.type.dims[0] ||
        dst.type.scale != zv.type.scale || dst.type.offset != zv.type.offset ||
        writers(G.operands[0]) != 1)
      return 0;
    for (size_t k = at + 1; k < j; k++)
      for (size_t i = 0; i < insts_[k].operands.size(); i++)
        if (M_.value(insts_[k].operands[i]).root == dst.root) return 0;
    destOf.assign((size_t)per, -1);
    const Operand io{&idx};
    for (int64_t k = 0; k < idx.type.dims[0]; k++) {
      const int64_t e = idx.type.kind == ElemKind::Int64ITy ? constData<int64_t>(io)[k]
                                                            : (int64_t)constData<int32_t>(io)[k];
      if (e < 0 || e >= per || destOf[(size_t)e] >= 0) return 0;
      destOf[(size_t)e] = (int32_t)k;
    }
    return j;
  }

  // Transpose + BatchMatMul, optionally with the Gather `G` of single elements
  // (destOf as soleGatherOf fills it) and the InsertTensor `ins` of the gathered
  // rows folded in.
  Error matmulNt(const Instruction &T, const Instruction &I, MI355XFunction &out,
                 const Instruction *G = nullptr, const std::vector<int32_t> &destOf = {},
                 const Instruction *ins = nullptr) {
    Operand d = op(I, 0), s = op(I, 1), r = op(T, 1);
    const size_t B = (size_t)s.ty().dims[0], M = (size_t)s.ty().dims[1], K = (size_t)s.ty().dims[2],
                 N = (size_t)r.ty().dims[1];
    const S32To8 p = s32to8(s.ty().scale * r.ty().scale / d.ty().scale);
    const int32_t oo = d.ty().offset, lo = s.ty().offset, ro = r.ty().offset;
    if (G) {
      Operand picked = op(*G, 0);
      SliceDest sd{picked, 0, (size_t)picked.ty().dims[1]};
      if (ins) sd = sliceDest(*ins);
      const size_t map = gen_.addI32(destOf);
      out.launches.push_back(
          {"mi355x_batch_matmul_nt_select_i8", I.name + "+" + G->name + (ins ? "+" + ins->name : ""),
           strFormat(" B=%zu M=%zu K=%zu N=%zu picked=%zu stride=%zu offset=%zu", B, M, K, N,
                     (size_t)picked.ty().dims[1], sd.pitch, sd.offset) +
               kv("out_offset", oo) + kv("lhs_offset", lo) + kv("rhs_offset", ro) + kv("out_pre", p.pre) +
               kv("out_post", p.post) + kv("out_scale", p.scale),
           [=](const DeviceBindings &b) {
             return mi355x_batch_matmul_nt_select_i8(
                 (int8_t *)sd.wide.ptr(b) + sd.offset, (const int8_t *)s.ptr(b), (const int8_t *)r.ptr(b),
                 B, M, K, N, oo, lo, ro, p.pre, p.post, p.scale, (const int32_t *)(b.generated + map),
                 sd.pitch, b.stream);
           }});
      return Error::success();
    }
    out.launches.push_back({"mi355x_batch_matmul_nt_i8", I.name,
                            strFormat(" B=%zu M=%zu K=%zu N=%zu", B, M, K, N) + kv("out_offset", oo) +
                                kv("lhs_offset", lo) + kv("rhs_offset", ro) + kv("out_pre", p.pre) +
                                kv("out_post", p.post) + kv("out_scale", p.scale),
                            [=](const DeviceBindings &b) {
                              return mi355x_batch_matmul_nt_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b),
                                                               (const int8_t *)r.ptr(b), B, M, K, N, oo, lo,
                                                               ro, p.pre, p.post, p.scale, b.stream);
                            }});
    return Error::success();
  }

  Error softmax(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), s = op(I, 1);
    CHECK_OP(d.ty().kind == ElemKind::FloatTy && s.ty().kind == ElemKind::FloatTy, "needs float tensors");
    CHECK_OP(s.ty().dims.size() == 2 && d.ty().dims == s.ty().dims, "needs equal 2-D shapes");
    const size_t rows = (size_t)s.ty().dims[0], cols = (size_t)s.ty().dims[1];
    out.launches.push_back({"mi355x_softmax_f32", I.name, strFormat(" rows=%zu cols=%zu", rows, cols),
                            [=](const DeviceBindings &b) {
                              return mi355x_softmax_f32((float *)d.ptr(b), (const float *)s.ptr(b), rows,
                                                        cols, b.stream);
                            }});
    return Error::success();
  }

  template <typename T> const T *constData(const Operand &o) const {
    return reinterpret_cast<const T *>(M_.constantsImage().data() + o.v->offset);
  }

  // pointer into the scratch part of the generated region; the base is only
  // known once every instruction has been seen
  std::function<uint8_t *(const DeviceBindings &)> scratchPtr(size_t rel) {
    auto base = scratchBasePtr_;
    return [base, rel](const DeviceBindings &b) { return b.generated + *base + rel; };
  }

  // The matrix-core launch just emitted multiplies [M x K] by [K x N] (per
  // group): when the library would split its K loop over workgroups given a
  // workspace, it gets one of its own (launches of one function may run side by
  // side), zero-filled once when the function is loaded.
  void planSplitK(MI355XFunction &out, size_t M, size_t N, size_t K, size_t groups) {
    if (!opts_.splitK) return;
    size_t bytes = 0;
    if (mi355x_gemm_splitk_workspace_bytes(M, N, K, groups, 0, &bytes) != MI355X_OK || bytes == 0)
      return;
    KernelLaunch &l = out.launches.back();
    l.workspaceRel = gen_.addScratch(bytes);
    l.workspaceBytes = bytes;
    l.scratchBase = scratchBasePtr_;
    l.params += strFormat(" splitk_workspace=%zu", bytes);
    auto p = scratchPtr(l.workspaceRel);
    out.setup.push_back({"mi355x_fill_u8", l.inst + ".splitk_workspace", strFormat(" bytes=%zu", bytes),
                         [=](const DeviceBindings &b) { return mi355x_fill_u8(p(b), 0, bytes, b.stream); }});
  }

  // Where a lookup reads a table and how far apart its rows are. A constant
  // table whose rows take 33..63 bytes is copied once, at load time, to rows 64
  // bytes apart: memory is fetched in 64-byte pieces, a 36-byte row at a 36-byte
  // pitch straddles two of them more often than not, and at 64 bytes it never
  // does. Costs 64/inLine of the table's size in device memory.
  struct TableView {
    std::function<const uint8_t *(const DeviceBindings &)> ptr;
    size_t pitch;
  };
  TableView tableView(const Operand &data, size_t rows, size_t inLine, MI355XFunction &out) {
    // (tables whose copy would pass 8 GiB keep their packed rows)
    if (!opts_.padTableRows || data.v->category != SymbolCategory::Constant || inLine <= 32 ||
        inLine >= 64 || rows == 0 || rows > ((size_t)8 << 30) / 64)
      return {[data](const DeviceBindings &b) { return (const uint8_t *)data.ptr(b); }, inLine};
    auto it = paddedTables_.find(data.v);
    if (it == paddedTables_.end()) {
      constexpr size_t kPitch = 64;
      auto dst = scratchPtr(gen_.addScratch(rows * kPitch));
      out.setup.push_back({"mi355x_insert_rows", data.v->name + ".pad_rows",
                           strFormat(" rows=%zu row_bytes=%zu pitch=%zu", rows, inLine, kPitch),
                           [=](const DeviceBindings &b) {
                             return mi355x_insert_rows(dst(b), data.ptr(b), rows, inLine, kPitch, 0,
                                                       b.stream);
                           }});
      it = paddedTables_.emplace(data.v, TableView{[dst](const DeviceBindings &b) {
                                                     return (const uint8_t *)dst(b);
                                                   },
                                                   kPitch}).first;
    }
    return it->second;
  }

  static bool wideKind(ElemKind k) { return k == ElemKind::Int16QTy || k == ElemKind::Int32QTy; }

  Error quantize(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), s = op(I, 1);
    CHECK_OP((d.ty().kind == ElemKind::Int8QTy || wideKind(d.ty().kind)) &&
                 s.ty().kind == ElemKind::FloatTy,
             "needs float -> i8, i16 or i32, has %s -> %s", s.ty().str().c_str(),
             d.ty().str().c_str());
    CHECK_OP(d.ty().size() == s.ty().size(), "size mismatch");
    const size_t n = (size_t)d.ty().size();
    const float sc = d.ty().scale;
    const int32_t off = d.ty().offset;
    if (wideKind(d.ty().kind)) {
      const bool w16 = d.ty().kind == ElemKind::Int16QTy;
      out.launches.push_back({w16 ? "mi355x_quantize_i16" : "mi355x_quantize_i32", I.name,
                              strFormat(" n=%zu scale=%.9g offset=%d", n, (double)sc, off),
                              [=](const DeviceBindings &b) {
                                return w16 ? mi355x_quantize_i16((int16_t *)d.ptr(b), (const float *)s.ptr(b),
                                                                 n, sc, off, b.stream)
                                           : mi355x_quantize_i32((int32_t *)d.ptr(b), (const float *)s.ptr(b),
                                                                 n, sc, off, b.stream);
                              }});
      return Error::success();
    }
    out.launches.push_back({"mi355x_quantize_i8", I.name,
                            strFormat(" n=%zu scale=%.9g offset=%d", n, (double)sc, off),
                            [=](const DeviceBindings &b) {
                              return mi355x_quantize_i8((int8_t *)d.ptr(b), (const float *)s.ptr(b),
                                                        n, sc, off, b.stream);
                            }});
    return Error::success();
  }

  Error dequantize(const Instruction &I, MI355XFunction &out, const Instruction *sig = nullptr,
                   const Instruction *smax = nullptr) {
    Operand d = op(I, 0), s = op(I, 1);
    CHECK_OP(d.ty().kind == ElemKind::FloatTy &&
                 (s.ty().kind == ElemKind::Int8QTy || (wideKind(s.ty().kind) && !sig)),
             "needs i8, i16 or i32 -> float, has %s -> %s", s.ty().str().c_str(),
             d.ty().str().c_str());
    CHECK_OP(d.ty().size() == s.ty().size(), "size mismatch");
    const size_t n = (size_t)d.ty().size();
    const float sc = s.ty().scale;
    const int32_t off = s.ty().offset;
    if (wideKind(s.ty().kind)) {
      const bool w16 = s.ty().kind == ElemKind::Int16QTy;
      out.launches.push_back({w16 ? "mi355x_dequantize_i16" : "mi355x_dequantize_i32", I.name,
                              strFormat(" n=%zu scale=%.9g offset=%d", n, (double)sc, off),
                              [=](const DeviceBindings &b) {
                                return w16 ? mi355x_dequantize_i16((float *)d.ptr(b), (const int16_t *)s.ptr(b),
                                                                   n, sc, off, b.stream)
                                           : mi355x_dequantize_i32((float *)d.ptr(b), (const int32_t *)s.ptr(b),
                                                                   n, sc, off, b.stream);
                              }});
      return Error::success();
    }
    if (sig) {
      Operand y = op(*sig, 0);
      out.launches.push_back({"mi355x_dequantize_sigmoid", I.name + "+" + sig->name,
                              strFormat(" n=%zu scale=%.9g offset=%d", n, (double)sc, off),
                              [=](const DeviceBindings &b) {
                                return mi355x_dequantize_sigmoid((float *)y.ptr(b), (const int8_t *)s.ptr(b),
                                                                 n, sc, off, b.stream);
                              }});
      return Error::success();
    }
    if (smax) {
      Operand y = op(*smax, 0);
      const size_t rows = (size_t)d.ty().dims[0], cols = (size_t)d.ty().dims[1];
      out.launches.push_back({"mi355x_dequantize_softmax", I.name + "+" + smax->name,
                              strFormat(" rows=%zu cols=%zu scale=%.9g offset=%d", rows, cols, (double)sc, off),
                              [=](const DeviceBindings &b) {
                                return mi355x_dequantize_softmax((float *)y.ptr(b), (const int8_t *)s.ptr(b),
                                                                 rows, cols, sc, off, b.stream);
                              }});
      return Error::success();
    }
    out.launches.push_back({"mi355x_dequantize_i8", I.name,
                            strFormat(" n=%zu scale=%.9g offset=%d", n, (double)sc, off),
                            [=](const DeviceBindings &b) {
                              return mi355x_dequantize_i8((float *)d.ptr(b), (const int8_t *)s.ptr(b),
                                                          n, sc, off, b.stream);
                            }});
    return Error::success();
  }

  Error rescale(const Instruction &I, MI355XFunction &out, const Instruction *ins = nullptr) {
    Operand d = op(I, 0), s = op(I, 1);
    CHECK_OP(d.ty().kind == s.ty().kind &&
                 (d.ty().kind == ElemKind::Int8QTy || (wideKind(d.ty().kind) && !ins)),
             "needs i8 -> i8, i16 -> i16 or i32 -> i32");
    CHECK_OP(d.ty().size() == s.ty().size(), "size mismatch");
    const size_t n = (size_t)d.ty().size();
    const S32To8 p = s32to8(s.ty().scale / d.ty().scale);
    const int32_t oo = d.ty().offset, io = s.ty().offset;
    if (wideKind(d.ty().kind)) {
      CHECK_OP(shiftsOk(p), "scales %g -> %g give a shift outside [0, 31]", (double)s.ty().scale,
               (double)d.ty().scale);
      const bool w16 = d.ty().kind == ElemKind::Int16QTy;
      out.launches.push_back(
          {w16 ? "mi355x_rescale_i16" : "mi355x_rescale_i32", I.name,
           strFormat(" n=%zu", n) + kv("out_offset", oo) + kv("in_offset", io) + kv("pre", p.pre) +
               kv("post", p.post) + kv("scale", p.scale),
           [=](const DeviceBindings &b) {
             return w16 ? mi355x_rescale_i16((int16_t *)d.ptr(b), (const int16_t *)s.ptr(b), n, oo, io,
                                             p.pre, p.post, p.scale, b.stream)
                        : mi355x_rescale_i32((int32_t *)d.ptr(b), (const int32_t *)s.ptr(b), n, oo, io,
                                             p.pre, p.post, p.scale, b.stream);
           }});
      return Error::success();
    }
    if (ins) {
      const SliceDest sd = sliceDest(*ins);
      const size_t rows = (size_t)d.ty().dims[0], cols = (size_t)d.ty().dims[1];
      out.launches.push_back(
          {"mi355x_rescale_rows_i8", I.name + "+" + ins->name,
           strFormat(" rows=%zu cols=%zu stride=%zu offset=%zu", rows, cols, sd.pitch, sd.offset) +
               kv("out_offset", oo) + kv("in_offset", io) + kv("pre", p.pre) + kv("post", p.post) +
               kv("scale", p.scale),
           [=](const DeviceBindings &b) {
             return mi355x_rescale_rows_i8((int8_t *)sd.wide.ptr(b) + sd.offset, (const int8_t *)s.ptr(b),
                                           rows, cols, sd.pitch, oo, io, p.pre, p.post, p.scale, b.stream);
           }});
      return Error::success();
    }
    out.launches.push_back(
        {"mi355x_rescale_i8", I.name,
         strFormat(" n=%zu", n) + kv("out_offset", oo) + kv("in_offset", io) +
             kv("pre", p.pre) + kv("post", p.post) + kv("scale", p.scale),
         [=](const DeviceBindings &b) {
           return mi355x_rescale_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), n, oo, io,
                                    p.pre, p.post, p.scale, b.stream);
         }});
    return Error::success();
  }

  static bool biasKindOk(ElemKind k) { return k == ElemKind::Int32QTy || k == ElemKind::Int8QTy; }

  Error fc(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), s = op(I, 1), w = op(I, 2), bi = op(I, 3);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && s.ty().kind == ElemKind::Int8QTy &&
                 w.ty().kind == ElemKind::Int8QTy && biasKindOk(bi.ty().kind),
             "needs i8 input, weights and output and an i32 or i8 bias");
    CHECK_OP(s.ty().dims.size() == 2 && w.ty().dims.size() == 2 && d.ty().dims.size() == 2 &&
                 bi.ty().dims.size() == 1,
             "needs 2-D input, weights and output and a 1-D bias");
    const size_t M = (size_t)s.ty().dims[0], K = (size_t)s.ty().dims[1], N = (size_t)w.ty().dims[1];
    CHECK_OP((size_t)w.ty().dims[0] == K && (size_t)d.ty().dims[0] == M &&
                 (size_t)d.ty().dims[1] == N && (size_t)bi.ty().dims[0] == N,
             "shape mismatch: %s x %s + %s -> %s", s.ty().str().c_str(), w.ty().str().c_str(),
             bi.ty().str().c_str(), d.ty().str().c_str());
    const float mm = s.ty().scale * w.ty().scale;
    const S32To8 bp = s32to8(bi.ty().scale / mm), opp = s32to8(mm / d.ty().scale);
    const int bias8 = bi.ty().kind == ElemKind::Int8QTy;
    const int32_t oo = d.ty().offset, io = s.ty().offset, wo = w.ty().offset, bo = bi.ty().offset;
    auto work = scratchPtr(gen_.addScratch(K * N));
    const bool wConst = w.v->category == SymbolCategory::Constant;
    const bool sums = wConst && opts_.precomputeWeightRowSums && io != 0;
    auto sumPtr = scratchPtr(sums ? gen_.addScratch(N * 4) : 0);
    if (wConst) {
      out.setup.push_back({"mi355x_transpose2d_i8", I.name, strFormat(" rows=%zu cols=%zu", K, N),
                           [=](const DeviceBindings &b) {
                             return mi355x_transpose2d_i8((int8_t *)work(b), (const int8_t *)w.ptr(b),
                                                          K, N, b.stream);
                           }});
      if (sums)
        out.setup.push_back({"mi355x_rowsum_i8", I.name, strFormat(" rows=%zu K=%zu", N, K),
                             [=](const DeviceBindings &b) {
                               return mi355x_rowsum_i8((int32_t *)sumPtr(b), (const int8_t *)work(b),
                                                       N, K, b.stream);
                             }});
    }
    const int repack = wConst ? 0 : 1;
    out.launches.push_back(
        {"mi355x_fc_i8", I.name,
         strFormat(" M=%zu K=%zu N=%zu", M, K, N) + kv("out_offset", oo) + kv("in_offset", io) +
             kv("weights_offset", wo) + kv("bias_offset", bo) + kv("bias_pre", bp.pre) +
             kv("bias_post", bp.post) + kv("bias_scale", bp.scale) + kv("out_pre", opp.pre) +
             kv("out_post", opp.post) + kv("out_scale", opp.scale) + kv("bias_is_i8", bias8) +
             kv("repack", repack) + kv("row_sums", sums),
         [=](const DeviceBindings &b) {
           return mi355x_fc_i8_opts((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), (const int8_t *)w.ptr(b),
                               (int8_t *)work(b), repack, bi.ptr(b), bias8, M, K, N, oo, io, wo, bo,
                               bp.pre, bp.post, bp.scale, opp.pre, opp.post, opp.scale,
                               sums ? (const int32_t *)sumPtr(b) : nullptr, b.stream, &b.opts);
         }});
    return Error::success();
  }

  Error matmul(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), l = op(I, 1), r = op(I, 2);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && l.ty().kind == ElemKind::Int8QTy &&
                 r.ty().kind == ElemKind::Int8QTy,
             "needs i8 operands");
    CHECK_OP(l.ty().dims.size() == 2 && r.ty().dims.size() == 2 && d.ty().dims.size() == 2,
             "needs 2-D operands");
    const size_t M = (size_t)l.ty().dims[0], K = (size_t)l.ty().dims[1], N = (size_t)r.ty().dims[1];
    CHECK_OP((size_t)r.ty().dims[0] == K && (size_t)d.ty().dims[0] == M && (size_t)d.ty().dims[1] == N,
             "shape mismatch");
    const S32To8 p = s32to8(l.ty().scale * r.ty().scale / d.ty().scale);
    const int32_t oo = d.ty().offset, lo = l.ty().offset, ro = r.ty().offset;
    auto work = scratchPtr(gen_.addScratch(K * N));
    const bool rConst = r.v->category == SymbolCategory::Constant;
    if (rConst)
      out.setup.push_back({"mi355x_transpose2d_i8", I.name, strFormat(" rows=%zu cols=%zu", K, N),
                           [=](const DeviceBindings &b) {
                             return mi355x_transpose2d_i8((int8_t *)work(b), (const int8_t *)r.ptr(b),
                                                          K, N, b.stream);
                           }});
    const int repack = rConst ? 0 : 1;
    out.launches.push_back(
        {"mi355x_matmul_i8", I.name,
         strFormat(" M=%zu K=%zu N=%zu", M, K, N) + kv("out_offset", oo) + kv("lhs_offset", lo) +
             kv("rhs_offset", ro) + kv("out_pre", p.pre) + kv("out_post", p.post) +
             kv("out_scale", p.scale) + kv("repack", repack),
         [=](const DeviceBindings &b) {
           return mi355x_matmul_i8_opts((int8_t *)d.ptr(b), (const int8_t *)l.ptr(b), (const int8_t *)r.ptr(b),
                                   (int8_t *)work(b), repack, M, K, N, oo, lo, ro, p.pre, p.post,
                                   p.scale, b.stream, &b.opts);
         }});
    return Error::success();
  }

  Error rwqfc(const Instruction &I, MI355XFunction &out, const Instruction *reluI = nullptr) {
    Operand d = op(I, 0), s = op(I, 1), w = op(I, 2), bi = op(I, 3), sc = op(I, 4), of = op(I, 5);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && s.ty().kind == ElemKind::Int8QTy &&
                 w.ty().kind == ElemKind::Int8QTy && biasKindOk(bi.ty().kind),
             "needs i8 input, weights and output and an i32 or i8 bias");
    CHECK_OP(sc.ty().kind == ElemKind::FloatTy && of.ty().kind == ElemKind::Int32ITy,
             "needs float scales and int32 offsets");
    CHECK_OP(sc.v->category == SymbolCategory::Constant && of.v->category == SymbolCategory::Constant &&
                 w.v->category == SymbolCategory::Constant,
             "weights, scales and offsets must be constants");
    CHECK_OP(s.ty().dims.size() == 2 && w.ty().dims.size() == 2 && d.ty().dims.size() == 2,
             "needs 2-D input, weights and output");
    const size_t M = (size_t)s.ty().dims[0], K = (size_t)s.ty().dims[1], N = (size_t)w.ty().dims[0];
    CHECK_OP((size_t)w.ty().dims[1] == K && (size_t)d.ty().dims[0] == M &&
                 (size_t)d.ty().dims[1] == N && (size_t)bi.ty().size() == N &&
                 (size_t)sc.ty().size() == N && (size_t)of.ty().size() == N,
             "shape mismatch: %s x %s^T + %s -> %s", s.ty().str().c_str(), w.ty().str().c_str(),
             bi.ty().str().c_str(), d.ty().str().c_str());
    const float *scales = constData<float>(sc);
    const int32_t *offsets = constData<int32_t>(of);
    std::vector<int32_t> bpre(N), bpost(N), bscale(N), opre(N), opost(N), oscale(N);
    bool allZero = true;
    for (size_t j = 0; j < N; j++) {
      const float mm = s.ty().scale * scales[j];
      const S32To8 bp = s32to8(bi.ty().scale / mm), opp = s32to8(mm / d.ty().scale);
      bpre[j] = bp.pre; bpost[j] = bp.post; bscale[j] = bp.scale;
      opre[j] = opp.pre; opost[j] = opp.post; oscale[j] = opp.scale;
      allZero = allZero && offsets[j] == 0;
      // the kernels shift by these amounts: what the scalar parameters are held
      // to at every entry point holds for each row's too
      CHECK_OP(shiftsOk(bp) && shiftsOk(opp),
               "row %zu: scales %g (input) x %g (weights), %g (bias), %g (output) give a "
               "shift outside [0, 31]", j, (double)s.ty().scale, (double)scales[j],
               (double)bi.ty().scale, (double)d.ty().scale);
    }
    const size_t o0 = gen_.addI32(bpre), o1 = gen_.addI32(bpost), o2 = gen_.addI32(bscale),
                 o3 = gen_.addI32(opre), o4 = gen_.addI32(opost), o5 = gen_.addI32(oscale);
    const int bias8 = bi.ty().kind == ElemKind::Int8QTy;
    const int32_t oo = d.ty().offset, io = s.ty().offset, bo = bi.ty().offset;
    const int hint = bi.v->category == SymbolCategory::Constant
                         ? requantHintFor(K, io, oo, offsets, constData<uint8_t>(bi), bias8, nullptr, bo,
                                          bpre, bpost, bscale, opre, opost, oscale)
                         : 0;
    const bool sums = opts_.precomputeWeightRowSums && io != 0;
    auto sumPtr = scratchPtr(sums ? gen_.addScratch(N * 4) : 0);
    if (sums)
      out.setup.push_back({"mi355x_rowsum_i8", I.name, strFormat(" rows=%zu K=%zu", N, K),
                           [=](const DeviceBindings &b) {
                             return mi355x_rowsum_i8((int32_t *)sumPtr(b), (const int8_t *)w.ptr(b), N,
                                                     K, b.stream);
                           }});
    if (reluI) {
      // the kernel's result keeps the FullyConnected's scale and offset; the
      // Relu stage maps it to the Relu's output type
      Operand rd = op(*reluI, 0);
      const S32To8 rp = s32to8(d.ty().scale / rd.ty().scale);
      const int32_t ro = rd.ty().offset;
      out.launches.push_back(
          {"mi355x_rwq_fc_relu_i8", I.name,
           strFormat(" M=%zu K=%zu N=%zu", M, K, N) + kv("fc_offset", oo) + kv("in_offset", io) +
               kv("bias_offset", bo) + kv("bias_is_i8", bias8) + kv("weights_offsets_all_zero", allZero) +
               kv("row_sums", sums) + kv("relu_offset", ro) + kv("relu_pre", rp.pre) +
               kv("relu_post", rp.post) + kv("relu_scale", rp.scale) + vecStr("bias_pre", bpre) +
               vecStr("bias_post", bpost) + vecStr("bias_scale", bscale) + vecStr("out_pre", opre) +
               vecStr("out_post", opost) + vecStr("out_scale", oscale),
           [=](const DeviceBindings &b) {
             auto g = [&](size_t o) { return (const int32_t *)(b.generated + o); };
             return mi355x_rwq_fc_relu_i8_opts((int8_t *)rd.ptr(b), (const int8_t *)s.ptr(b),
                                          (const int8_t *)w.ptr(b), bi.ptr(b), bias8,
                                          (const int32_t *)of.ptr(b), g(o0), g(o1), g(o2), g(o3), g(o4),
                                          g(o5), M, K, N, oo, io, bo, allZero ? 1 : 0,
                                          sums ? (const int32_t *)sumPtr(b) : nullptr, ro, rp.pre,
                                          rp.post, rp.scale, b.stream, &b.opts);
           }});
      out.launches.back().requantHint = hint;
      planSplitK(out, M, N, K, 1);
      return Error::success();
    }
    out.launches.push_back(
        {"mi355x_rwq_fc_i8", I.name,
         strFormat(" M=%zu K=%zu N=%zu", M, K, N) + kv("out_offset", oo) + kv("in_offset", io) +
             kv("bias_offset", bo) + kv("bias_is_i8", bias8) + kv("weights_offsets_all_zero", allZero) +
             kv("row_sums", sums) + vecStr("bias_pre", bpre) + vecStr("bias_post", bpost) +
             vecStr("bias_scale", bscale) + vecStr("out_pre", opre) + vecStr("out_post", opost) +
             vecStr("out_scale", oscale),
         [=](const DeviceBindings &b) {
           auto g = [&](size_t o) { return (const int32_t *)(b.generated + o); };
           return mi355x_rwq_fc_i8_opts((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), (const int8_t *)w.ptr(b),
                                   bi.ptr(b), bias8, (const int32_t *)of.ptr(b), g(o0), g(o1), g(o2),
                                   g(o3), g(o4), g(o5), M, K, N, oo, io, bo, allZero ? 1 : 0,
                                   sums ? (const int32_t *)sumPtr(b) : nullptr, b.stream, &b.opts);
         }});
    out.launches.back().requantHint = hint;
    planSplitK(out, M, N, K, 1);
    return Error::success();
  }

  // ChannelwiseQuantizedConvolution over NTHWC tensors. Integer attributes:
  // {KT, KH, KW, strideT, strideH, strideW, padNear, padFar, padTop, padBottom,
  // padLeft, padRight, group, activation}.
  Error conv3d(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), s = op(I, 1), f = op(I, 2), bi = op(I, 3);
    Operand fs = op(I, 4), fo = op(I, 5), bs = op(I, 6), bo = op(I, 7);
    CHECK_OP(I.iattrs.size() == 14, "the 3-D form expects 14 integer attributes");
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && s.ty().kind == ElemKind::Int8QTy &&
                 f.ty().kind == ElemKind::Int8QTy && biasKindOk(bi.ty().kind),
             "needs i8 input, filter and output and an i32 or i8 bias");
    CHECK_OP(s.ty().dims.size() == 5 && f.ty().dims.size() == 5 && d.ty().dims.size() == 5,
             "needs NTHWC input and output and an [OC,KT,KH,KW,IC/group] filter");
    const auto &a = I.iattrs;
    for (int i = 0; i < 13; i++) CHECK_OP(a[i] >= 0 && a[i] < (1 << 20), "attribute %d out of range", i);
    mi355x_conv3d_geom g;
    g.N = (int32_t)s.ty().dims[0]; g.IT = (int32_t)s.ty().dims[1]; g.IH = (int32_t)s.ty().dims[2];
    g.IW = (int32_t)s.ty().dims[3]; g.IC = (int32_t)s.ty().dims[4];
    g.OT = (int32_t)d.ty().dims[1]; g.OH = (int32_t)d.ty().dims[2]; g.OW = (int32_t)d.ty().dims[3];
    g.OC = (int32_t)d.ty().dims[4];
    g.KT = (int32_t)a[0]; g.KH = (int32_t)a[1]; g.KW = (int32_t)a[2];
    g.strideT = (int32_t)a[3]; g.strideH = (int32_t)a[4]; g.strideW = (int32_t)a[5];
    g.padN = (int32_t)a[6]; g.padT = (int32_t)a[8]; g.padL = (int32_t)a[10];
    g.group = (int32_t)a[12];
    const int32_t act = (int32_t)a[13];
    CHECK_OP(g.KT > 0 && g.KH > 0 && g.KW > 0 && g.strideT > 0 && g.strideH > 0 && g.strideW > 0 &&
                 g.group > 0, "invalid kernel, stride or group");
    CHECK_OP(g.IC % g.group == 0 && g.OC % g.group == 0, "channels not divisible by group");
    CHECK_OP(f.ty().dims[0] == g.OC && f.ty().dims[1] == g.KT && f.ty().dims[2] == g.KH &&
                 f.ty().dims[3] == g.KW && f.ty().dims[4] == g.IC / g.group,
             "filter %s does not match", f.ty().str().c_str());
    CHECK_OP(d.ty().dims[0] == g.N && bi.ty().size() == g.OC, "batch or bias size mismatch");
    // calculate3DConvPoolOutputDims (reference include/glow/Graph/Nodes.h)
    const int64_t ot = (g.IT + a[6] + a[7] - g.KT) / g.strideT + 1;
    const int64_t oh = (g.IH + a[8] + a[9] - g.KH) / g.strideH + 1;
    const int64_t ow = (g.IW + a[10] + a[11] - g.KW) / g.strideW + 1;
    CHECK_OP(ot == g.OT && oh == g.OH && ow == g.OW,
             "output %s does not match the computed %lld x %lld x %lld", d.ty().str().c_str(),
             (long long)ot, (long long)oh, (long long)ow);
    CHECK_OP(act == NONE || act == RELU || act == CLIP || act == LEAKY_RELU,
             "fused activation %d is not supported for quantized types", act);
    std::vector<int32_t> actArgs(3, 0);
    if (act == CLIP) {
      CHECK_OP(I.fattrs.size() == 2, "fused Clip needs {min, max}");
      actArgs[0] = quantizeI32(I.fattrs[0], d.ty().scale, d.ty().offset);
      actArgs[1] = quantizeI32(I.fattrs[1], d.ty().scale, d.ty().offset);
    } else if (act == LEAKY_RELU) {
      CHECK_OP(I.fattrs.size() == 1, "fused LeakyRelu needs {alpha}");
      const S32To8 p = s32to8(I.fattrs[0]);
      actArgs = {p.pre, p.post, p.scale};
    } else {
      CHECK_OP(I.fattrs.empty(), "activation takes no arguments");
    }
    CHECK_OP(fs.ty().kind == ElemKind::FloatTy && bs.ty().kind == ElemKind::FloatTy &&
                 fo.ty().kind == ElemKind::Int32ITy && bo.ty().kind == ElemKind::Int32ITy,
             "needs float scales and int32 offsets");
    CHECK_OP(fs.v->category == SymbolCategory::Constant && fo.v->category == SymbolCategory::Constant &&
                 bs.v->category == SymbolCategory::Constant && bo.v->category == SymbolCategory::Constant,
             "filter/bias scales and offsets must be constants");
    const size_t OC = (size_t)g.OC;
    CHECK_OP((size_t)fs.ty().size() == OC && (size_t)fo.ty().size() == OC &&
                 (size_t)bs.ty().size() == OC && (size_t)bo.ty().size() == OC,
             "per-channel vectors must have one entry per output channel");
    const float *fsc = constData<float>(fs), *bsc = constData<float>(bs);
    std::vector<int32_t> bpre(OC), bpost(OC), bscale(OC), opre(OC), opost(OC), oscale(OC);
    for (size_t c = 0; c < OC; c++) {
      const float mm = s.ty().scale * fsc[c];
      const S32To8 bp = s32to8(bsc[c] / mm), opp = s32to8(mm / d.ty().scale);
      bpre[c] = bp.pre; bpost[c] = bp.post; bscale[c] = bp.scale;
      opre[c] = opp.pre; opost[c] = opp.post; oscale[c] = opp.scale;
      CHECK_OP(shiftsOk(bp) && shiftsOk(opp), "channel %zu: the scales give a shift outside [0, 31]", c);
    }
    const size_t o0 = gen_.addI32(bpre), o1 = gen_.addI32(bpost), o2 = gen_.addI32(bscale),
                 o3 = gen_.addI32(opre), o4 = gen_.addI32(opost), o5 = gen_.addI32(oscale);
    const int bias8 = bi.ty().kind == ElemKind::Int8QTy;
    const int32_t oo = d.ty().offset, io = s.ty().offset;
    out.launches.push_back(
        {"mi355x_cwq_conv3d_i8", I.name,
         strFormat(" N=%d IT=%d IH=%d IW=%d IC=%d OT=%d OH=%d OW=%d OC=%d KT=%d KH=%d KW=%d sT=%d sH=%d "
                   "sW=%d padN=%d padT=%d padL=%d group=%d", g.N, g.IT, g.IH, g.IW, g.IC, g.OT, g.OH,
                   g.OW, g.OC, g.KT, g.KH, g.KW, g.strideT, g.strideH, g.strideW, g.padN, g.padT,
                   g.padL, g.group) +
             kv("out_offset", oo) + kv("in_offset", io) + kv("act", act) + vecStr("act_args", actArgs) +
             kv("bias_is_i8", bias8),
         [=](const DeviceBindings &b) {
           auto gp = [&](size_t o) { return (const int32_t *)(b.generated + o); };
           return mi355x_cwq_conv3d_i8((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), (const int8_t *)f.ptr(b),
                                       bi.ptr(b), bias8, &g, oo, io, (const int32_t *)fo.ptr(b),
                                       (const int32_t *)bo.ptr(b), gp(o0), gp(o1), gp(o2), gp(o3), gp(o4),
                                       gp(o5), act, actArgs.data(), b.stream);
         }});
    return Error::success();
  }

  // quantI: the Quantize whose result this convolution alone reads (it is
  // emitted here: folded into the space-to-depth pass, or as its own launch
  // in front of everything else)
  Error conv(const Instruction &I, MI355XFunction &out, bool channelwise,
             const Instruction *addI = nullptr, const Instruction *reluI = nullptr,
             const Instruction *quantI = nullptr) {
    Operand d = op(I, 0), s = op(I, 1), f = op(I, 2), bi = op(I, 3);
    CHECK_OP((int)I.iattrs.size() == ConvAttrs::kCount, "expects %d integer attributes",
             ConvAttrs::kCount);
    CHECK_OP(d.ty().kind == ElemKind::Int8QTy && s.ty().kind == ElemKind::Int8QTy &&
                 f.ty().kind == ElemKind::Int8QTy && biasKindOk(bi.ty().kind),
             "needs i8 input, filter and output and an i32 or i8 bias");
    CHECK_OP(s.ty().dims.size() == 4 && f.ty().dims.size() == 4 && d.ty().dims.size() == 4,
             "needs NHWC input and output and an [OC,KH,KW,IC/group] filter");
    const auto &a = I.iattrs;
    mi355x_conv_geom g;
    g.N = (int32_t)s.ty().dims[0]; g.IH = (int32_t)s.ty().dims[1];
    g.IW = (int32_t)s.ty().dims[2]; g.IC = (int32_t)s.ty().dims[3];
    g.OH = (int32_t)d.ty().dims[1]; g.OW = (int32_t)d.ty().dims[2]; g.OC = (int32_t)d.ty().dims[3];
    g.KH = (int32_t)a[0]; g.KW = (int32_t)a[1]; g.strideH = (int32_t)a[2]; g.strideW = (int32_t)a[3];
    g.padT = (int32_t)a[4]; g.padL = (int32_t)a[5];
    const int64_t padB = a[6], padR = a[7];
    g.group = (int32_t)a[8]; g.dilH = (int32_t)a[9]; g.dilW = (int32_t)a[10];
    const int32_t act = (int32_t)a[11];
    CHECK_OP(g.KH > 0 && g.KW > 0 && g.strideH > 0 && g.strideW > 0 && g.group > 0 && g.dilH > 0 &&
                 g.dilW > 0 && g.padT >= 0 && g.padL >= 0 && padB >= 0 && padR >= 0,
             "invalid kernel, stride, pad, group or dilation");
    CHECK_OP(g.IC % g.group == 0 && g.OC % g.group == 0, "channels not divisible by group");
    CHECK_OP(f.ty().dims[0] == g.OC && f.ty().dims[1] == g.KH && f.ty().dims[2] == g.KW &&
                 f.ty().dims[3] == g.IC / g.group,
             "filter %s does not match", f.ty().str().c_str());
    CHECK_OP(d.ty().dims[0] == g.N && bi.ty().size() == g.OC, "batch or bias size mismatch");
    // calculateConvPoolOutputDims (reference include/glow/Graph/Nodes.h / Utils)
    const int64_t oh = (g.IH + g.padT + padB - (g.KH - 1) * g.dilH - 1) / g.strideH + 1;
    const int64_t ow = (g.IW + g.padL + padR - (g.KW - 1) * g.dilW - 1) / g.strideW + 1;
    CHECK_OP(oh == g.OH && ow == g.OW, "output %s does not match the computed %lld x %lld",
             d.ty().str().c_str(), (long long)oh, (long long)ow);
    CHECK_OP(act == NONE || act == RELU || act == CLIP || act == LEAKY_RELU,
             "fused activation %d is not supported for quantized types", act);
    // emitConstQuantActivationArgs (LLVMIRGen.cpp:618-662)
    std::vector<int32_t> actArgs(3, 0);
    if (act == CLIP) {
      CHECK_OP(I.fattrs.size() == 2, "fused Clip needs {min, max}");
      actArgs[0] = quantizeI32(I.fattrs[0], d.ty().scale, d.ty().offset);
      actArgs[1] = quantizeI32(I.fattrs[1], d.ty().scale, d.ty().offset);
    } else if (act == LEAKY_RELU) {
      CHECK_OP(I.fattrs.size() == 1, "fused LeakyRelu needs {alpha}");
      const S32To8 p = s32to8(I.fattrs[0]);
      actArgs = {p.pre, p.post, p.scale};
    } else {
      CHECK_OP(I.fattrs.empty(), "activation takes no arguments");
    }
    CHECK_OP(f.v->category == SymbolCategory::Constant, "filter must be a constant");
    const size_t OC = (size_t)g.OC, Kf = (size_t)g.KH * g.KW * (g.IC / g.group);
    const int bias8 = bi.ty().kind == ElemKind::Int8QTy;
    const int32_t oo = d.ty().offset, io = s.ty().offset;
    const bool sums = opts_.precomputeWeightRowSums && io != 0;
    auto sumPtr = scratchPtr(sums ? gen_.addScratch(OC * 4) : 0);
    if (sums)
      out.setup.push_back({"mi355x_rowsum_i8", I.name, strFormat(" rows=%zu K=%zu", OC, Kf),
                           [=](const DeviceBindings &b) {
                             return mi355x_rowsum_i8((int32_t *)sumPtr(b), (const int8_t *)f.ptr(b), OC,
                                                     Kf, b.stream);
                           }});
    std::string geomStr = strFormat(" N=%d IH=%d IW=%d IC=%d OH=%d OW=%d OC=%d KH=%d KW=%d sH=%d sW=%d "
                                    "padT=%d padL=%d dH=%d dW=%d group=%d",
                                    g.N, g.IH, g.IW, g.IC, g.OH, g.OW, g.OC, g.KH, g.KW, g.strideH,
                                    g.strideW, g.padT, g.padL, g.dilH, g.dilW, g.group);
    if (quantI && !channelwise) MI355X_RETURN_IF_ERR(quantize(*quantI, out));
    if (!channelwise) {
      const float mm = s.ty().scale * f.ty().scale;
      const S32To8 bp = s32to8(bi.ty().scale / mm), opp = s32to8(mm / d.ty().scale);
      const int32_t fo = f.ty().offset, bo = bi.ty().offset;
      out.launches.push_back(
          {"mi355x_conv2d_i8", I.name,
           geomStr + kv("out_offset", oo) + kv("in_offset", io) + kv("filter_offset", fo) +
               kv("bias_offset", bo) + kv("bias_pre", bp.pre) + kv("bias_post", bp.post) +
               kv("bias_scale", bp.scale) + kv("out_pre", opp.pre) + kv("out_post", opp.post) +
               kv("out_scale", opp.scale) + kv("act", act) + vecStr("act_args", actArgs) +
               kv("bias_is_i8", bias8) + kv("row_sums", sums),
           [=](const DeviceBindings &b) {
             return mi355x_conv2d_i8_opts((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b), (const int8_t *)f.ptr(b),
                                     bi.ptr(b), bias8, &g, oo, io, fo, bo, bp.pre, bp.post, bp.scale,
                                     opp.pre, opp.post, opp.scale, act, actArgs.data(),
                                     sums ? (const int32_t *)sumPtr(b) : nullptr, b.stream, &b.opts);
           }});
      return Error::success();
    }
    Operand fs = op(I, 4), fo = op(I, 5), bs = op(I, 6), bo = op(I, 7);
    CHECK_OP(fs.ty().kind == ElemKind::FloatTy && bs.ty().kind == ElemKind::FloatTy &&
                 fo.ty().kind == ElemKind::Int32ITy && bo.ty().kind == ElemKind::Int32ITy,
             "needs float scales and int32 offsets");
    CHECK_OP(fs.v->category == SymbolCategory::Constant && fo.v->category == SymbolCategory::Constant &&
                 bs.v->category == SymbolCategory::Constant && bo.v->category == SymbolCategory::Constant,
             "filter/bias scales and offsets must be constants");
    CHECK_OP((size_t)fs.ty().size() == OC && (size_t)fo.ty().size() == OC &&
                 (size_t)bs.ty().size() == OC && (size_t)bo.ty().size() == OC,
             "per-channel vectors must have one entry per output channel");
    const float *fsc = constData<float>(fs), *bsc = constData<float>(bs);
    const int32_t *fof = constData<int32_t>(fo);
    std::vector<int32_t> bpre(OC), bpost(OC), bscale(OC), opre(OC), opost(OC), oscale(OC);
    bool allZero = true;
    for (size_t c = 0; c < OC; c++) {
      const float mm = s.ty().scale * fsc[c];
      const S32To8 bp = s32to8(bsc[c] / mm), opp = s32to8(mm / d.ty().scale);
      bpre[c] = bp.pre; bpost[c] = bp.post; bscale[c] = bp.scale;
      opre[c] = opp.pre; opost[c] = opp.post; oscale[c] = opp.scale;
      allZero = allZero && fof[c] == 0;
      CHECK_OP(shiftsOk(bp) && shiftsOk(opp),
               "channel %zu: scales %g (input) x %g (filter), %g (bias), %g (output) give a "
               "shift outside [0, 31]", c, (double)s.ty().scale, (double)fsc[c], (double)bsc[c],
               (double)d.ty().scale);
    }
    const size_t o0 = gen_.addI32(bpre), o1 = gen_.addI32(bpost), o2 = gen_.addI32(bscale),
                 o3 = gen_.addI32(opre), o4 = gen_.addI32(opost), o5 = gen_.addI32(oscale);
    // (K: the longest contraction any form of this convolution runs: the
    // space-to-depth form pads the taps up to an even count per direction)
    auto convHint = [&](size_t k) {
      return bi.v->category == SymbolCategory::Constant
                 ? requantHintFor(k, io, oo, fof, constData<uint8_t>(bi), bias8,
                                  constData<int32_t>(bo), 0, bpre, bpost, bscale, opre, opost, oscale)
                 : 0;
    };
    // A stride-2 convolution over at most 4 channels (the first layer of an
    // image network) cannot feed the matrix cores 16 bytes at a time. Space-to-
    // depth by 2 turns it into a stride-1 convolution over 16 channels on a
    // half-size image: same sums, since padded taps meet (input == inOffset)
    // and padded filter entries equal the filter offset, both contributing 0.
    bool fitsI8 = true;
    for (size_t c = 0; c < OC; c++) fitsI8 = fitsI8 && fof[c] >= -128 && fof[c] <= 127;
    if (opts_.spaceToDepthStem && !addI && g.strideH == 2 && g.strideW == 2 && g.dilH == 1 &&
        g.dilW == 1 && g.group == 1 && g.IC * 4 <= 16 && fitsI8) {
      const int KH2 = (g.KH + 1) / 2, KW2 = (g.KW + 1) / 2, C2 = 16;
      const size_t BH = (size_t)g.OH + KH2 - 1, BW = (size_t)g.OW + KW2 - 1;
      const int8_t *F = constData<int8_t>(f);
      std::vector<int8_t> F2((size_t)OC * KH2 * KW2 * C2);
      for (size_t oc = 0; oc < OC; oc++)
        for (int bh = 0; bh < KH2; bh++)
          for (int bw = 0; bw < KW2; bw++)
            for (int ch = 0; ch < C2; ch++) {
              const int q = ch / g.IC, c = ch % g.IC;
              const int kh = 2 * bh + (q >> 1), kw = 2 * bw + (q & 1);
              int8_t v = (int8_t)fof[oc];
              if (ch < 4 * g.IC && kh < g.KH && kw < g.KW)
                v = F[((oc * g.KH + kh) * g.KW + kw) * g.IC + c];
              F2[((oc * KH2 + bh) * KW2 + bw) * C2 + ch] = v;
            }
      const size_t f2 = gen_.addBytes(F2);
      const size_t K2 = (size_t)KH2 * KW2 * C2;
      auto sPtr = scratchPtr(gen_.addScratch((size_t)g.N * BH * BW * C2));
      auto sum2 = scratchPtr(sums ? gen_.addScratch(OC * 4) : 0);
      if (sums)
        out.setup.push_back({"mi355x_rowsum_i8", I.name, strFormat(" rows=%zu K=%zu", OC, K2),
                             [=](const DeviceBindings &b) {
                               return mi355x_rowsum_i8((int32_t *)sum2(b), (const int8_t *)(b.generated + f2),
                                                       OC, K2, b.stream);
                             }});
      mi355x_conv_geom g2 = g;
      g2.IH = (int32_t)BH; g2.IW = (int32_t)BW; g2.IC = C2;
      g2.KH = KH2; g2.KW = KW2; g2.strideH = g2.strideW = 1; g2.padT = g2.padL = 0;
      Access priv;                       // the private image orders the two launches
      priv.root = -100 - (int)out.launches.size();
      const size_t N = (size_t)g.N, IH = (size_t)g.IH, IW = (size_t)g.IW, IC = (size_t)g.IC,
                   pT = (size_t)g.padT, pL = (size_t)g.padL;
      if (quantI && (IC == 3 || IC == 4) && op(*quantI, 1).ty().kind == ElemKind::FloatTy &&
          op(*quantI, 1).ty().size() == s.ty().size()) {
        // the float image is quantized while it is re-laid
        Operand qs = op(*quantI, 1);
        const float qscale = s.ty().scale;
        out.launches.push_back(
            {"mi355x_quantize_space_to_depth2_i8", quantI->name + "+" + I.name + ".s2d",
             strFormat(" N=%zu IH=%zu IW=%zu C=%zu padT=%zu padL=%zu BH=%zu BW=%zu Cout=%d scale=%.9g", N,
                       IH, IW, IC, pT, pL, BH, BW, C2, (double)qscale) + kv("offset", io) + kv("fill", io),
             [=](const DeviceBindings &b) {
               return mi355x_quantize_space_to_depth2_i8((int8_t *)sPtr(b), (const float *)qs.ptr(b), N,
                                                         IH, IW, IC, pT, pL, BH, BW, (size_t)C2, io,
                                                         qscale, io, b.stream);
             }});
      } else {
        if (quantI) MI355X_RETURN_IF_ERR(quantize(*quantI, out));
        out.launches.push_back(
            {"mi355x_space_to_depth2_i8", I.name + ".s2d",
             strFormat(" N=%zu IH=%zu IW=%zu C=%zu padT=%zu padL=%zu BH=%zu BW=%zu Cout=%d", N, IH, IW, IC,
                       pT, pL, BH, BW, C2) + kv("fill", io),
             [=](const DeviceBindings &b) {
               return mi355x_space_to_depth2_i8((int8_t *)sPtr(b), (const int8_t *)s.ptr(b), N, IH, IW, IC,
                                                pT, pL, BH, BW, (size_t)C2, io, b.stream);
             }});
      }
      out.launches.back().writes.push_back(priv);
      out.launches.push_back(
          {"mi355x_cwq_conv2d_i8", I.name,
           strFormat(" N=%d IH=%d IW=%d IC=%d OH=%d OW=%d OC=%d KH=%d KW=%d sH=1 sW=1 padT=0 padL=0 dH=1 "
                     "dW=1 group=1 space_to_depth=1", g2.N, g2.IH, g2.IW, g2.IC, g2.OH, g2.OW, g2.OC,
                     g2.KH, g2.KW) +
               kv("out_offset", oo) + kv("in_offset", io) + kv("act", act) + vecStr("act_args", actArgs) +
               kv("bias_is_i8", bias8) + kv("filter_offsets_all_zero", allZero) + kv("row_sums", sums) +
               vecStr("bias_pre", bpre) + vecStr("bias_post", bpost) + vecStr("bias_scale", bscale) +
               vecStr("out_pre", opre) + vecStr("out_post", opost) + vecStr("out_scale", oscale),
           [=](const DeviceBindings &b) {
             auto gp = [&](size_t o) { return (const int32_t *)(b.generated + o); };
             return mi355x_cwq_conv2d_i8_opts((int8_t *)d.ptr(b), (const int8_t *)sPtr(b),
                                         (const int8_t *)(b.generated + f2), bi.ptr(b), bias8, &g2, oo, io,
                                         (const int32_t *)fo.ptr(b), (const int32_t *)bo.ptr(b), gp(o0),
                                         gp(o1), gp(o2), gp(o3), gp(o4), gp(o5), act, actArgs.data(),
                                         allZero ? 1 : 0, sums ? (const int32_t *)sum2(b) : nullptr,
                                         b.stream, &b.opts);
           }});
      out.launches.back().requantHint = convHint(K2);
      planSplitK(out, (size_t)g2.N * g2.OH * g2.OW, (size_t)g2.OC, (size_t)K2, 1);
      out.launches.back().reads.push_back(priv);
      return Error::success();
    }
    if (quantI) MI355X_RETURN_IF_ERR(quantize(*quantI, out));
    if (addI) {
      const Instruction &A = *addI;
      const bool convIsLhs = A.operands[1] == I.operands[0];
      Operand sum = op(A, 0), res = op(A, convIsLhs ? 2 : 1);
      {
        const Instruction &I = A; // for the message
        CHECK_OP(sum.ty().kind == ElemKind::Int8QTy && res.ty().kind == ElemKind::Int8QTy &&
                     res.ty().size() == sum.ty().size(),
                 "needs i8 operands of one size");
      }
      mi355x_fused_add fa;
      const S32To8 cp = s32to8(d.ty().scale / sum.ty().scale), rp = s32to8(res.ty().scale / sum.ty().scale);
      fa.sum_offset = sum.ty().offset;
      fa.residual_offset = res.ty().offset;
      fa.conv_pre = cp.pre; fa.conv_post = cp.post; fa.conv_scale = cp.scale;
      fa.residual_pre = rp.pre; fa.residual_post = rp.post; fa.residual_scale = rp.scale;
      fa.relu = reluI ? 1 : 0;
      fa.dest_offset = 0; fa.dest_pre = 0; fa.dest_post = 0; fa.dest_scale = 1;
      Operand fin = sum;
      std::string name = I.name + "+" + A.name;
      if (reluI) {
        fin = op(*reluI, 0);
        {
          const Instruction &I = *reluI;
          CHECK_OP(fin.ty().kind == ElemKind::Int8QTy && fin.ty().size() == sum.ty().size(),
                   "needs an i8 result of the same size");
        }
        const S32To8 dp = s32to8(sum.ty().scale / fin.ty().scale);
        fa.dest_offset = fin.ty().offset;
        fa.dest_pre = dp.pre; fa.dest_post = dp.post; fa.dest_scale = dp.scale;
        name += "+" + reluI->name;
      }
      out.launches.push_back(
          {"mi355x_cwq_conv2d_add_i8", name,
           geomStr + kv("out_offset", oo) + kv("in_offset", io) + kv("act", act) +
               vecStr("act_args", actArgs) + kv("bias_is_i8", bias8) +
               kv("filter_offsets_all_zero", allZero) + kv("row_sums", sums) +
               kv("sum_offset", fa.sum_offset) + kv("residual_offset", fa.residual_offset) +
               kv("conv_pre", fa.conv_pre) + kv("conv_post", fa.conv_post) +
               kv("conv_scale", fa.conv_scale) + kv("residual_pre", fa.residual_pre) +
               kv("residual_post", fa.residual_post) + kv("residual_scale", fa.residual_scale) +
               kv("relu", fa.relu) + kv("relu_dest_offset", fa.dest_offset) +
               kv("relu_pre", fa.dest_pre) + kv("relu_post", fa.dest_post) +
               kv("relu_scale", fa.dest_scale),
           [=](const DeviceBindings &b) {
             auto gp = [&](size_t o) { return (const int32_t *)(b.generated + o); };
             return mi355x_cwq_conv2d_add_i8_opts(
                 (int8_t *)fin.ptr(b), (const int8_t *)s.ptr(b), (const int8_t *)f.ptr(b), bi.ptr(b),
                 bias8, &g, oo, io, (const int32_t *)fo.ptr(b), (const int32_t *)bo.ptr(b), gp(o0),
                 gp(o1), gp(o2), gp(o3), gp(o4), gp(o5), act, actArgs.data(), allZero ? 1 : 0,
                 sums ? (const int32_t *)sumPtr(b) : nullptr, (const int8_t *)res.ptr(b), &fa,
                 b.stream, &b.opts);
           }});
      out.launches.back().requantHint = convHint(Kf);
      planSplitK(out, (size_t)g.N * g.OH * g.OW, (size_t)g.OC / g.group, (size_t)Kf, (size_t)g.group);
      return Error::success();
    }
    out.launches.push_back(
        {"mi355x_cwq_conv2d_i8", I.name,
         geomStr + kv("out_offset", oo) + kv("in_offset", io) + kv("act", act) +
             vecStr("act_args", actArgs) + kv("bias_is_i8", bias8) +
             kv("filter_offsets_all_zero", allZero) + kv("row_sums", sums) + vecStr("bias_pre", bpre) +
             vecStr("bias_post", bpost) + vecStr("bias_scale", bscale) + vecStr("out_pre", opre) +
             vecStr("out_post", opost) + vecStr("out_scale", oscale),
         [=](const DeviceBindings &b) {
           auto gp = [&](size_t o) { return (const int32_t *)(b.generated + o); };
           return mi355x_cwq_conv2d_i8_opts((int8_t *)d.ptr(b), (const int8_t *)s.ptr(b),
                                       (const int8_t *)f.ptr(b), bi.ptr(b), bias8, &g, oo, io,
                                       (const int32_t *)fo.ptr(b), (const int32_t *)bo.ptr(b), gp(o0),
                                       gp(o1), gp(o2), gp(o3), gp(o4), gp(o5), act, actArgs.data(),
                                       allZero ? 1 : 0, sums ? (const int32_t *)sumPtr(b) : nullptr,
                                       b.stream, &b.opts);
         }});
    out.launches.back().requantHint = convHint(Kf);
    planSplitK(out, (size_t)g.N * g.OH * g.OW, (size_t)g.OC / g.group, (size_t)Kf, (size_t)g.group);
    return Error::success();
  }

  // The two other pooled-lookup forms of the CPU backend (fp32 throughout).
  Error otherLookups(const Instruction &I, MI355XFunction &out) {
    Operand d = op(I, 0), data = op(I, 1);
    CHECK_OP(d.ty().kind == ElemKind::FloatTy && d.ty().dims.size() == 2, "result must be 2-D float");
    CHECK_OP(data.ty().dims.size() == 2, "data must be 2-D");
    const size_t rows = (size_t)data.ty().dims[0], line = (size_t)data.ty().dims[1];
    if (I.kind == Kind::RowwiseQuantizedSparseLengthsWeightedSum) {
      Operand sc = op(I, 2), of = op(I, 3), w = op(I, 4), idx = op(I, 5), len = op(I, 6);
      CHECK_OP(elemSize(data.ty().kind) == 1 && !isFused(data.ty().kind), "data must be plain 8-bit rows");
      CHECK_OP(sc.ty().kind == ElemKind::FloatTy && of.ty().kind == ElemKind::FloatTy &&
                   w.ty().kind == ElemKind::FloatTy,
               "scales, offsets and weights must be float");
      CHECK_OP((size_t)sc.ty().size() == rows && (size_t)of.ty().size() == rows,
               "one scale and offset per row");
      CHECK_OP(idx.ty().kind == ElemKind::Int64ITy || idx.ty().kind == ElemKind::Int32ITy,
               "indices must be int64 or int32");
      CHECK_OP(len.ty().kind == ElemKind::Int32ITy && w.ty().size() == idx.ty().size(),
               "lengths must be int32; one weight per index");
      CHECK_OP(d.ty().dims[0] == len.ty().size() && (size_t)d.ty().dims[1] == line, "result shape mismatch");
      const size_t nIdx = (size_t)idx.ty().size(), segs = (size_t)len.ty().size();
      const int i64 = idx.ty().kind == ElemKind::Int64ITy;
      out.launches.push_back({"mi355x_rwq_slws", I.name,
                              strFormat(" rows=%zu line=%zu segments=%zu num_indices=%zu", rows, line, segs, nIdx) +
                                  kv("idx_is_64", i64),
                              [=](const DeviceBindings &b) {
                                return mi355x_rwq_slws_opts((float *)d.ptr(b), data.ptr(b), rows, (const float *)sc.ptr(b),
                                                       (const float *)of.ptr(b), (const float *)w.ptr(b), idx.ptr(b),
                                                       i64, nIdx, (const int32_t *)len.ptr(b), segs, line, b.stream, &b.opts);
                              }});
      return Error::success();
    }
    Operand w = op(I, 2), idx = op(I, 3), offs = op(I, 4);
    CHECK_OP(data.ty().kind == ElemKind::UInt8FusedQTy, "data must be ui8fused");
    CHECK_OP(w.ty().kind == ElemKind::FloatTy && idx.ty().kind == ElemKind::Int32ITy &&
                 offs.ty().kind == ElemKind::Int32ITy,
             "needs float weights and int32 indices and offsets");
    CHECK_OP(I.iattrs.size() == 1, "expects {hasEndOffset}");
    const int hasEnd = I.iattrs[0] != 0;
    const size_t segs = (size_t)offs.ty().size(), nIdx = (size_t)idx.ty().size();
    CHECK_OP(line > 8 && (size_t)d.ty().dims[1] == line - 8 && (size_t)d.ty().dims[0] + hasEnd == segs &&
                 w.ty().size() == idx.ty().size(),
             "shape mismatch");
    out.launches.push_back({"mi355x_embedding_bag_rowwise_offsets", I.name,
                            strFormat(" rows=%zu in_line=%zu segments=%zu num_indices=%zu", rows, line, segs, nIdx) +
                                kv("has_end_offset", hasEnd),
                            [=](const DeviceBindings &b) {
                              return mi355x_embedding_bag_rowwise_offsets_opts(
                                  d.ptr(b), 0, data.ptr(b), rows, MI355X_FUSED_U8_F32, w.ptr(b), 0,
                                  (const int32_t *)idx.ptr(b), nIdx, (const int32_t *)offs.ptr(b), segs, hasEnd,
                                  line, line - 8, 0, b.stream, &b.opts);
                            }});
    return Error::success();
  }

  // One pooled lookup followed by [ConvertTo,] Quantize and InsertTensor, each
  // intermediate read only by the next instruction.
  struct SlsChain {
    Operand data, idx, len, dest; // dest: the tensor the int8 rows are inserted into
    size_t colOffset = 0;         // where, in elements
    size_t length = 0;            // instructions in the chain
    int kind = 0, idx64 = 0, viaF16 = 0, acc16 = 0;
    size_t rows = 0, inLine = 0, cols = 0, segs = 0, nIdx = 0;
    float qScale = 1.0f;
    int32_t qOffset = 0;
  };

  bool matchSlsChain(size_t at, SlsChain &c) const {
    if (at + 2 >= insts_.size()) return false;
    const Instruction &S = insts_[at];
    if (S.kind != Kind::FusedRowwiseQuantizedSparseLengthsSum) return false;
    auto onlyReadBy = [&](int id, const Instruction &J) {
      return M_.value(id).category == SymbolCategory::Activation && readers(id) == 1 &&
             J.operands[1] == id;
    };
    size_t p = at + 1;
    int cur = S.operands[0];
    const Value &sd = M_.value(cur);
    if (sd.type.dims.size() != 2) return false;
    if (sd.type.kind == ElemKind::Float16Ty) {
      const Instruction &Cv = insts_[p];
      if (Cv.kind != Kind::ConvertTo || !onlyReadBy(cur, Cv)) return false;
      if (M_.value(Cv.operands[0]).type.kind != ElemKind::FloatTy) return false;
      cur = Cv.operands[0];
      p++;
      c.viaF16 = 1;
    } else if (sd.type.kind != ElemKind::FloatTy) {
      return false;
    }
    if (p + 1 >= insts_.size()) return false;
    const Instruction &Q = insts_[p], &Ins = insts_[p + 1];
    if (Q.kind != Kind::Quantize || !onlyReadBy(cur, Q)) return false;
    const Value &qv = M_.value(Q.operands[0]);
    if (qv.type.kind != ElemKind::Int8QTy) return false;
    if (Ins.kind != Kind::InsertTensor || !onlyReadBy(qv.id, Ins) || Ins.iattrs.size() != 1) return false;
    const Value &dv = M_.value(Ins.operands[0]);
    if (dv.type.kind != ElemKind::Int8QTy || dv.type.dims.size() != 2 || dv.id != dv.root) return false;
    if (dv.type.scale != qv.type.scale || dv.type.offset != qv.type.offset) return false;
    const Value &data = M_.value(S.operands[1]), &idx = M_.value(S.operands[2]),
                &len = M_.value(S.operands[3]);
    if (!isFused(data.type.kind) || data.type.dims.size() != 2) return false;
    bool fp16Scale = false, fourBit = false;
    switch (data.type.kind) {
    case ElemKind::UInt8FusedQTy: c.kind = MI355X_FUSED_U8_F32; break;
    case ElemKind::UInt8FusedFP16QTy: c.kind = MI355X_FUSED_U8_F16; fp16Scale = true; break;
    case ElemKind::UInt4FusedFP16QTy: c.kind = MI355X_FUSED_U4_F16; fp16Scale = fourBit = true; break;
    default: c.kind = MI355X_FUSED_U4_F32; fourBit = true; break;
    }
    if (fp16Scale && !c.viaF16) return false; // not a legal lookup: let slws() report it
    if (idx.type.kind != ElemKind::Int64ITy && idx.type.kind != ElemKind::Int32ITy) return false;
    if (len.type.kind != ElemKind::Int32ITy) return false;
    c.rows = (size_t)data.type.dims[0];
    c.inLine = (size_t)data.type.dims[1];
    c.cols = (size_t)sd.type.dims[1];
    c.segs = (size_t)len.type.size();
    c.nIdx = (size_t)idx.type.size();
    const size_t so = fp16Scale ? 4 : 8;
    if (c.inLine <= so || (c.inLine - so) * (fourBit ? 2 : 1) != c.cols) return false;
    if ((size_t)sd.type.dims[0] != c.segs || c.segs > 4096 || c.segs == 0) return false;
    if ((size_t)dv.type.dims[0] != c.segs) return false;
    if (qv.type.size() != sd.type.size()) return false;
    c.colOffset = (size_t)Ins.iattrs[0];
    if (Ins.iattrs[0] < 0 || c.colOffset + c.cols > (size_t)dv.type.dims[1]) return false;
    c.idx64 = idx.type.kind == ElemKind::Int64ITy;
    c.acc16 = !S.iattrs.empty() && S.iattrs[0] != 0 && fp16Scale;
    c.qScale = qv.type.scale;
    c.qOffset = qv.type.offset;
    c.data = opOf(data);
    c.idx = opOf(idx);
    c.len = opOf(len);
    c.dest = opOf(dv);
    c.length = p + 2 - at;
    return true;
  }

  // Consecutive lookup chains of one shape feeding one tensor become a single
  // multi-table launch. Returns the number of instructions consumed (0: none).
  size_t multiSls(size_t at, MI355XFunction &out) {
    std::vector<SlsChain> group;
    size_t pos = at;
    for (;;) {
      SlsChain c;
      if (!matchSlsChain(pos, c)) break;
      if (!group.empty()) {
        const SlsChain &g = group[0];
        if (c.kind != g.kind || c.idx64 != g.idx64 || c.viaF16 != g.viaF16 || c.acc16 != g.acc16 ||
            c.inLine != g.inLine || c.cols != g.cols || c.segs != g.segs || c.qScale != g.qScale ||
            c.qOffset != g.qOffset || c.dest.v != g.dest.v)
          break;
      }
      group.push_back(c);
      pos += c.length;
      if (group.size() == 1024) break;
    }
    if (group.empty()) return 0;
    const size_t n = group.size();
    const SlsChain g = group[0];
    size_t maxRows = 0;
    for (const auto &c : group) maxRows = std::max(maxRows, c.rows);
    // tables of one group have one row size, so all of them are re-laid or none
    std::vector<TableView> views;
    for (const auto &c : group) views.push_back(tableView(c.data, c.rows, c.inLine, out));
    const size_t pitch = views[0].pitch;
    auto tabPtr = scratchPtr(gen_.addScratch(n * sizeof(mi355x_sls_table)));
    std::vector<std::function<uint8_t *(const DeviceBindings &)>> offs;
    size_t nDerived = 0;
    for (const auto &c : group) {
      offs.push_back(derivedOffsets(c.len, out));
      nDerived += offs.back() ? 1 : 0;
    }
    const size_t stride = (size_t)g.dest.ty().dims[1];
    const std::string name = insts_[at].name + (n > 1 ? "..." + insts_[pos - 1].name : "");
    // the table array holds device addresses: written once the buffers are bound
    out.setup.push_back({"mi355x_memcpy_h2d", name, strFormat(" tables=%zu", n),
                         [=](const DeviceBindings &b) {
                           std::vector<mi355x_sls_table> t(n);
                           for (size_t i = 0; i < n; i++) {
                             t[i].data = views[i].ptr(b);
                             t[i].indices = group[i].idx.ptr(b);
                             t[i].lengths = (const int32_t *)group[i].len.ptr(b);
                             t[i].dest = group[i].dest.ptr(b) + group[i].colOffset;
                             t[i].data_rows = group[i].rows;
                             t[i].num_indices = group[i].nIdx;
                             t[i].bag_offsets = offs[i] ? (const int32_t *)offs[i](b) : nullptr;
                           }
                           int rc = mi355x_memcpy_h2d(tabPtr(b), t.data(), n * sizeof(mi355x_sls_table),
                                                      b.stream);
                           if (rc == MI355X_OK) rc = mi355x_stream_sync(b.stream);
                           return rc;
                         }});
    const int outKind = g.viaF16 ? MI355X_SLS_OUT_I8_VIA_F16 : MI355X_SLS_OUT_I8;
    out.launches.push_back(
        {"mi355x_frwq_sls_multi", name,
         strFormat(" tables=%zu max_rows=%zu in_line=%zu out_line=%zu segments=%zu stride=%zu", n, maxRows,
                   pitch, g.cols, g.segs, stride) +
             kv("kind", g.kind) + kv("idx_is_64", g.idx64) + kv("out_kind", outKind) +
             strFormat(" out_scale=%.9g", (double)g.qScale) + kv("out_offset", g.qOffset) +
             kv("fp16_accum", g.acc16) + kv("bag_offsets_from_host", (long long)nDerived),
         [=](const DeviceBindings &b) {
           return mi355x_frwq_sls_multi_opts((const mi355x_sls_table *)tabPtr(b), n, maxRows, g.kind, g.idx64,
                                        g.segs, pitch, g.cols, outKind, g.qScale, g.qOffset, stride,
                                        g.acc16, b.stream, &b.opts);
         }});
    return pos - at;
  }

  // Whether an instruction of any function of the module writes `root` or a view of it.
  bool writtenInModule(int root) const {
    auto writes = [&](const std::vector<Instruction> &insts) {
      for (const auto &I : insts)
        if (!I.operands.empty() && M_.validId(I.operands[0]) &&
            M_.value(I.operands[0]).root == root)
          return true;
      return false;
    };
    if (writes(insts_)) return true;
    for (const auto &f : M_.functions())
      if (f && writes(f->instructions())) return true;
    return false;
  }

  // The bag positions of a lookup whose lengths are an input of the function
  // (a placeholder no instruction writes): a scratch vector the device manager
  // fills when it uploads the lengths. Empty function: read the lengths.
  std::function<uint8_t *(const DeviceBindings &)> derivedOffsets(const Operand &len,
                                                                 MI355XFunction &out) {
    if (!opts_.deriveBagOffsets || len.v->category != SymbolCategory::Placeholder ||
        len.v->id != len.v->root)
      return nullptr;
    // written on the device, directly or through a view, by this function or by
    // another one the module holds so far: the host's copy would be stale
    if (writtenInModule(len.v->id)) return nullptr;
    auto it = derived_.find(len.v->id);
    if (it != derived_.end()) return out.derivedBagOffsets[it->second].ptr;
    const size_t segs = (size_t)len.ty().size();
    MI355XFunction::DerivedBagOffsets d;
    d.lengths = len.v->name;
    d.segments = segs;
    d.ptr = scratchPtr(gen_.addScratch((segs + 1) * sizeof(int32_t)));
    derived_[len.v->id] = out.derivedBagOffsets.size();
    out.derivedBagOffsets.push_back(d);
    return d.ptr;
  }

  Error slws(const Instruction &I, MI355XFunction &out, bool weighted) {
    Operand d = op(I, 0), data = op(I, 1);
    Operand w = weighted ? op(I, 2) : Operand{nullptr, nullptr};
    Operand idx = op(I, weighted ? 3 : 2), len = op(I, weighted ? 4 : 3);
    CHECK_OP(isFused(data.ty().kind) && data.ty().dims.size() == 2,
             "data must be a 2-D fused-rowwise tensor, has %s", data.ty().str().c_str());
    int kind = MI355X_FUSED_U8_F32;
    bool fp16Scale = false, fourBit = false;
    switch (data.ty().kind) {
    case ElemKind::UInt8FusedQTy: kind = MI355X_FUSED_U8_F32; break;
    case ElemKind::UInt8FusedFP16QTy: kind = MI355X_FUSED_U8_F16; fp16Scale = true; break;
    case ElemKind::UInt4FusedFP16QTy: kind = MI355X_FUSED_U4_F16; fp16Scale = fourBit = true; break;
    default: kind = MI355X_FUSED_U4_F32; fourBit = true; break;
    }
    const ElemKind dk = d.ty().kind;
    CHECK_OP(dk == ElemKind::FloatTy || dk == ElemKind::Float16Ty, "result must be float or float16");
    // type legality of the reference (lib/Backends/Interpreter/Interpreter.cpp:526-567)
    if (fp16Scale)
      CHECK_OP(dk == ElemKind::Float16Ty, "fp16-scale data needs a float16 result");
    ElemKind wk = dk; // the lowered plain sum uses a splat of the result kind
    if (weighted) {
      wk = w.ty().kind;
      CHECK_OP(wk == ElemKind::FloatTy || wk == ElemKind::Float16Ty, "weights must be float or float16");
      if (!fp16Scale)
        CHECK_OP(wk == dk, "fp32-scale data needs weights and result of the same kind");
    }
    CHECK_OP(idx.ty().kind == ElemKind::Int64ITy || idx.ty().kind == ElemKind::Int32ITy,
             "indices must be int64 or int32");
    CHECK_OP(len.ty().kind == ElemKind::Int32ITy, "lengths must be int32");
    CHECK_OP(d.ty().dims.size() == 2 && d.ty().dims[0] == len.ty().size(),
             "result must be [lengths x columns]");
    if (weighted) CHECK_OP(w.ty().size() == idx.ty().size(), "weights and indices differ in size");
    const size_t rows = (size_t)data.ty().dims[0], inLine = (size_t)data.ty().dims[1];
    const size_t outLine = (size_t)d.ty().dims[1];
    const size_t so = fp16Scale ? 4 : 8;
    CHECK_OP(inLine > so && (inLine - so) * (fourBit ? 2 : 1) == outLine,
             "row of %zu bytes does not hold %zu columns", inLine, outLine);
    const bool acc16 = !I.iattrs.empty() && I.iattrs[0] != 0 && fp16Scale;
    const size_t nIdx = (size_t)idx.ty().size(), segs = (size_t)len.ty().size();
    const int out16 = dk == ElemKind::Float16Ty, w16 = wk == ElemKind::Float16Ty;
    const int idx64 = idx.ty().kind == ElemKind::Int64ITy;
    const TableView table = tableView(data, rows, inLine, out);
    const size_t pitch = table.pitch;
    if (auto offs = derivedOffsets(len, out)) {
      out.launches.push_back(
          {"mi355x_frwq_slws_offsets", I.name,
           strFormat(" rows=%zu in_line=%zu out_line=%zu segments=%zu num_indices=%zu", rows, pitch,
                     outLine, segs, nIdx) +
               kv("kind", kind) + kv("out_is_f16", out16) + kv("weighted", weighted) +
               kv("weights_are_f16", w16) + kv("idx_is_64", idx64) + kv("fp16_accum", acc16) +
               " bag_offsets=host(" + len.v->name + ")",
           [=](const DeviceBindings &b) {
             return mi355x_frwq_slws_offsets_opts(d.ptr(b), out16, table.ptr(b), rows, kind,
                                             weighted ? (const void *)w.ptr(b) : nullptr, w16,
                                             idx.ptr(b), idx64, nIdx, (const int32_t *)offs(b), segs,
                                             pitch, outLine, acc16 ? 1 : 0, b.stream, &b.opts);
           }});
      return Error::success();
    }
    out.launches.push_back(
        {"mi355x_frwq_slws", I.name,
         strFormat(" rows=%zu in_line=%zu out_line=%zu segments=%zu num_indices=%zu", rows, pitch,
                   outLine, segs, nIdx) +
             kv("kind", kind) + kv("out_is_f16", out16) + kv("weighted", weighted) +
             kv("weights_are_f16", w16) + kv("idx_is_64", idx64) + kv("fp16_accum", acc16),
         [=](const DeviceBindings &b) {
           return mi355x_frwq_slws_opts(d.ptr(b), out16, table.ptr(b), rows, kind,
                                   weighted ? (const void *)w.ptr(b) : nullptr, w16, idx.ptr(b), idx64,
                                   nIdx, (const int32_t *)len.ptr(b), segs, pitch, outLine,
                                   acc16 ? 1 : 0, b.stream, &b.opts);
         }});
    return Error::success();
  }

  const Module &M_;
  const std::vector<Instruction> &insts_;
  int function_;
  BackendOptions opts_;
  Generated gen_;
  size_t scratchBase_ = 0, genTotal_ = 0;
  std::shared_ptr<size_t> scratchBasePtr_ = std::make_shared<size_t>(0);
  std::shared_ptr<std::vector<size_t>> actOff_;   // value id -> place in the activations region
  std::map<int, std::pair<bool, bool>> io_; // value id -> (read, written)
  std::map<const Value *, TableView> paddedTables_;
  std::map<int, size_t> derived_; // lengths value id -> index in derivedBagOffsets
  std::vector<char> absorbed_; // instructions folded into the launch of an earlier one
};

constexpr int Compiler::kArity[];

} // namespace

Expected<std::unique_ptr<MI355XFunction>> MI355XBackend::compile(const Function &F,
                                                                 const BackendOptions &opts) const {
  const Module &M = *F.module();
  Compiler C(M, F.instructions(), F.index(), opts);
  auto fn = std::unique_ptr<MI355XFunction>(new MI355XFunction(RuntimeBundle(), F.name()));
  Error e = C.run(*fn);
  if (e) return e;
  for (const auto &I : F.instructions()) {
    if (I.operands.empty() || !M.validId(I.operands[0])) continue;
    const Value &root = M.value(M.value(I.operands[0]).root);
    if (root.category == SymbolCategory::Placeholder &&
        std::find(fn->writtenPlaceholders.begin(), fn->writtenPlaceholders.end(), root.name) ==
            fn->writtenPlaceholders.end())
      fn->writtenPlaceholders.push_back(root.name);
  }
  RuntimeBundle rb;
  rb.constantWeightVarsMemSize = M.constantsSize();
  rb.mutableWeightVarsMemSize = M.mutableSize();
  rb.activationsMemSize = fn->activationsBytes;
  rb.generatedConstantsMemSize = C.generatedTotal();
  for (int id = 0; id < M.numValues(); id++) {
    const Value &v = M.value(id);
    if (v.category == SymbolCategory::Activation && v.function != F.index()) continue;
    RuntimeSymbolInfo si;
    si.size = v.type.sizeInBytes();
    si.offset = v.category == SymbolCategory::Activation ? (*fn->activationOffsets)[(size_t)id]
                                                         : v.offset;
    si.type = v.type;
    si.symbolCategory = v.category;
    auto it = C.io().find(id);
    if (it != C.io().end() && v.category == SymbolCategory::Placeholder) {
      si.input = it->second.first;
      si.output = it->second.second;
    }
    rb.symbolTable[v.name] = si;
  }
  fn->setRuntimeBundle(std::move(rb));
  return fn;
}

bool MI355XBackend::isOpSupported(const Module &M, const Instruction &I, std::string *why) const {
  std::vector<Instruction> one{I};
  Compiler C(M, one, -1, BackendOptions());
  MI355XFunction scratch(RuntimeBundle(), "probe");
  Error e = C.run(scratch);
  if (e && why) *why = e.message();
  return !e;
}

bool MI355XBackend::shouldLower(Kind k) const {
  switch (k) {
  case Kind::FullyConnected:
  case Kind::Convolution:
  case Kind::RowwiseQuantizedFullyConnected:
  case Kind::ChannelwiseQuantizedConvolution:
  case Kind::Relu:
  case Kind::Clip:
  case Kind::LeakyRelu:
  case Kind::SoftMax:
    return false;
  default:
    return true;
  }
}

bool MI355XBackend::supportsFusedActivation(Kind parent, FusedActivation act) const {
  if (parent != Kind::Convolution && parent != Kind::ChannelwiseQuantizedConvolution) return false;
  return act == RELU || act == CLIP || act == LEAKY_RELU;
}

unsigned MI355XBackend::numDevices() {
  int n = 0;
  if (mi355x_num_devices(&n) != MI355X_OK) return 0;
  return n < 0 ? 0u : (unsigned)n;
}

int KernelLaunch::launch(const DeviceBindings &b) const {
  if (!tunable || (tile < 0 && requantHint == 0 && workspaceBytes == 0)) return run(b);
  // the launch's own tile, hint and workspace travel with the call, nothing is left set
  DeviceBindings mine = b;
  mine.opts.gemm_tile = tile;
  mine.opts.requant_hint = requantHint;
  if (workspaceBytes && scratchBase) {
    mine.opts.workspace = b.generated + *scratchBase + workspaceRel;
    mine.opts.workspace_bytes = workspaceBytes;
  }
  return run(mine);
}

MI355XFunction::~MI355XFunction() { dropGraph(); }

void MI355XFunction::dropGraph() {
  if (graph_) {
    mi355x_graph_destroy(graph_);
    graph_ = nullptr;
  }
}

static bool sameBindings(const DeviceBindings &a, const DeviceBindings &b) {
  return a.constants == b.constants && a.generated == b.generated &&
         a.mutableMem == b.mutableMem && a.activations == b.activations;
}

static bool launchesConflict(const KernelLaunch &early, const KernelLaunch &late) {
  for (const auto &w : early.writes) {
    for (const auto &r : late.reads) if (w.overlaps(r)) return true;
    for (const auto &x : late.writes) if (w.overlaps(x)) return true;
  }
  for (const auto &r : early.reads)
    for (const auto &w : late.writes) if (r.overlaps(w)) return true;
  return false;
}

// The launches form a dependence DAG (read/write sets). Each launch is put on
// the stream ("lane") of its latest predecessor when it can continue that
// chain, on an unused lane otherwise; dependences across lanes become event
// waits. Captured this way the graph runs independent chains side by side.
Error MI355XFunction::captureGraph(const DeviceBindings &b, const std::vector<void *> &sideStreams) {
  dropGraph();
  if (launches.empty()) return Error::success();
  if (!b.stream)
    return MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "graph capture needs a created stream");
  const size_t n = launches.size();
  size_t nLanes = sideStreams.size() + 1;
  // Direct predecessors only: a conflicting launch that is already an ancestor
  // of a later predecessor is ordered through it (memory shared by values whose
  // lives do not meet makes a launch conflict with every earlier owner of its
  // bytes; recorded as edges, those made graphs the runtime could not walk).
  std::vector<std::vector<size_t>> preds(n);
  {
    const size_t words = (n + 63) / 64;
    std::vector<std::vector<uint64_t>> anc(n, std::vector<uint64_t>(words, 0));
    for (size_t i = 0; i < n; i++) {
      for (size_t j = i; j-- > 0;) {
        if ((anc[i][j / 64] >> (j % 64)) & 1) continue;
        if (!launchesConflict(launches[j], launches[i])) continue;
        preds[i].push_back(j);
        anc[i][j / 64] |= 1ull << (j % 64);
        for (size_t w = 0; w < words; w++) anc[i][w] |= anc[j][w];
      }
      std::reverse(preds[i].begin(), preds[i].end());   // ascending, as the lane choice expects
    }
  }
  // Lanes. A launch hands its lane to the successor with the longest chain of
  // launches still behind it, so the critical path runs down one stream and
  // only the shorter branches pay for an event wait.
  std::vector<int> height(n, 1), depth(n, 1);
  std::vector<long long> heir(n, -1);
  for (size_t i = n; i-- > 0;)
    for (size_t p : preds[i])
      if (height[i] + 1 > height[p]) height[p] = height[i] + 1;
  for (size_t i = 0; i < n; i++)
    for (size_t p : preds[i]) {
      if (depth[p] + 1 > depth[i]) depth[i] = depth[p] + 1;
      if (heir[p] < 0 || height[i] > height[(size_t)heir[p]]) heir[p] = (long long)i;
    }
  // The waits between side streams must not run in a circle (stream 1 waits
  // for 2, 2 for 3, 3 for 1, each at a different point of the recording): the
  // runtime's end-of-capture walk over the streams that joined a capture does
  // not come back from such a ring. The capturing stream is exempt (every side
  // stream forks from it and joins it). When the assignment below produces a
  // ring it is redone with one lane fewer; with a single side stream there is
  // none.
  std::vector<int> lane(n, 0);
  std::vector<long long> last;
  for (;; nLanes--) {
    std::fill(lane.begin(), lane.end(), 0);
    last.assign(nLanes, -1);                  // last launch put on each lane
    for (size_t i = 0; i < n; i++) {
      int pick = -1;
      // the heir continues; the heir of several launches follows the deepest
      long long from = -1;
      for (size_t p : preds[i])
        if (heir[p] == (long long)i && (from < 0 || depth[p] >= depth[(size_t)from])) from = (long long)p;
      if (from >= 0) pick = lane[(size_t)from];
      if (pick < 0)
        for (size_t l = 0; l < nLanes && pick < 0; l++)
          if (last[l] < 0) pick = (int)l;                                  // an unused lane
      // lanes whose last launch still waits for its heir are kept for it
      auto kept = [&](size_t l) { return heir[(size_t)last[l]] > (long long)i; };
      if (pick < 0)
        for (auto it = preds[i].rbegin(); it != preds[i].rend() && pick < 0; ++it)
          if (last[(size_t)lane[*it]] == (long long)*it && !kept((size_t)lane[*it]))
            pick = lane[*it];                                              // behind a predecessor
      if (pick < 0)
        for (size_t l = 0; l < nLanes; l++)                                // idle longest
          if (!kept(l) && (pick < 0 || last[l] < last[(size_t)pick])) pick = (int)l;
      if (pick < 0) pick = preds[i].empty() ? 0 : lane[preds[i].back()];
      lane[i] = pick;
      last[(size_t)pick] = (long long)i;
    }
    if (nLanes <= 2) break;
    std::vector<std::vector<char>> waits(nLanes, std::vector<char>(nLanes, 0));
    for (size_t i = 0; i < n; i++)
      for (size_t p : preds[i])
        if (lane[p] != lane[i] && lane[p] != 0 && lane[i] != 0) waits[(size_t)lane[p]][(size_t)lane[i]] = 1;
    for (size_t k = 1; k < nLanes; k++)       // transitive closure over the side lanes
      for (size_t a = 1; a < nLanes; a++)
        for (size_t c = 1; c < nLanes; c++)
          if (waits[a][k] && waits[k][c]) waits[a][c] = 1;
    bool ring = false;
    for (size_t a = 1; a < nLanes; a++) ring = ring || waits[a][a];
    if (!ring) break;
  }
  // which launches need an event recorded behind them
  std::vector<char> needsEvent(n, 0);
  for (size_t i = 0; i < n; i++)
    for (size_t p : preds[i])
      if (lane[p] != lane[i]) needsEvent[p] = 1;
  for (size_t l = 1; l < nLanes; l++)
    if (last[l] >= 0) needsEvent[(size_t)last[l]] = 1;                   // joined at the end
  std::vector<void *> events(n, nullptr);
  void *fork = nullptr;
  auto streamOf = [&](int l) { return l == 0 ? b.stream : sideStreams[(size_t)l - 1]; };
  auto cleanup = [&] {
    if (fork) mi355x_event_destroy(fork);
    for (void *e : events) if (e) mi355x_event_destroy(e);
  };
  int rc = mi355x_event_create(&fork);
  for (size_t i = 0; i < n && rc == MI355X_OK; i++)
    if (needsEvent[i]) rc = mi355x_event_create(&events[i]);
  if (rc != MI355X_OK) {
    cleanup();
    return MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "%s", mi355x_last_error());
  }
  if (mi355x_graph_begin_capture(b.stream) != MI355X_OK) {
    cleanup();
    return MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "%s", mi355x_last_error());
  }
  std::string failed;
  std::vector<char> forked(nLanes, 0);
  forked[0] = 1;
  rc = mi355x_event_record(fork, b.stream);
  for (size_t i = 0; i < n && rc == MI355X_OK; i++) {
    void *st = streamOf(lane[i]);
    if (!forked[(size_t)lane[i]]) {         // a side lane joins the capture
      rc = mi355x_stream_wait_event(st, fork);
      forked[(size_t)lane[i]] = 1;
    }
    for (size_t p : preds[i])
      if (lane[p] != lane[i] && rc == MI355X_OK) rc = mi355x_stream_wait_event(st, events[p]);
    if (rc != MI355X_OK) break;
    DeviceBindings bb = b;
    bb.stream = st;
    rc = launches[i].launch(bb);
    if (rc != MI355X_OK) {
      failed = launches[i].kernel + " (" + launches[i].inst + "): " + mi355x_last_error();
      break;
    }
    if (needsEvent[i]) rc = mi355x_event_record(events[i], st);
  }
  // every side lane flows back into the capturing stream
  for (size_t l = 1; l < nLanes && rc == MI355X_OK; l++)
    if (last[l] >= 0 && forked[l]) rc = mi355x_stream_wait_event(b.stream, events[(size_t)last[l]]);
  if (rc != MI355X_OK && failed.empty()) failed = mi355x_last_error();
  mi355x_graph *g = nullptr;
  const int rc2 = mi355x_graph_end_capture(b.stream, &g);
  cleanup();
  if (rc != MI355X_OK) {
    if (g) mi355x_graph_destroy(g);
    return MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "%s", failed.c_str());
  }
  if (rc2 != MI355X_OK)
    return MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "%s", mi355x_last_error());
  graph_ = g;
  graphBindings_ = b;
  return Error::success();
}

Error MI355XFunction::execute(ExecutionContext *ctx) {
  DeviceBindings *b = ctx ? ctx->getDeviceBindings() : nullptr;
  if (!b)
    return MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR,
                           "function %s executed without device bindings", name_.c_str());
  if (graph_ && sameBindings(*b, graphBindings_)) {
    if (mi355x_graph_launch(graph_, b->stream) != MI355X_OK)
      return MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "%s", mi355x_last_error());
    return Error::success();
  }
  for (const auto &l : launches) {
    const int rc = l.launch(*b);
    if (rc != MI355X_OK)
      return MI355X_MAKE_ERR(rc == MI355X_ERR_NOT_SUPPORTED ? ErrorCode::DEVICE_FEATURE_NOT_SUPPORTED
                                                            : ErrorCode::RUNTIME_ERROR,
                             "%s (%s): %s", l.kernel.c_str(), l.inst.c_str(), mi355x_last_error());
  }
  return Error::success();
}

std::vector<int32_t> MI355XFunction::bagOffsets(const int32_t *lengths, size_t n, size_t segments) {
  std::vector<int32_t> o(segments + 1, 0);
  int64_t sum = 0;
  for (size_t i = 0; i < segments; i++) {
    if (i < n && lengths[i] > 0) sum = std::min<int64_t>(sum + lengths[i], 0x7fffffff);
    o[i + 1] = (int32_t)sum;
  }
  return o;
}

std::string MI355XFunction::describe() const {
  std::ostringstream os;
  os << "function " << name_ << " constants=" << bundle_.constantWeightVarsMemSize
     << " generated=" << bundle_.generatedConstantsMemSize
     << " mutable=" << bundle_.mutableWeightVarsMemSize
     << " activations=" << bundle_.activationsMemSize << "\n";
  for (const auto &l : setup) os << "setup " << l.kernel << " inst=" << l.inst << l.params << "\n";
  auto accesses = [&](const char *k, const std::vector<Access> &v) {
    // value ids (views by their root) and the byte range inside a row, -1 = all
    for (const char *part : {"", "_lo", "_hi"}) {
      os << " " << k << part << "=[";
      for (size_t i = 0; i < v.size(); i++)
        os << (i ? "," : "") << (*part == 0 ? (long long)v[i].root : part[1] == 'l' ? v[i].lo : v[i].hi);
      os << "]";
    }
  };
  for (const auto &l : launches) {
    os << "launch " << l.kernel << " inst=" << l.inst << " level=" << l.level << " tile=" << l.tile << " requant_hint=" << l.requantHint
       << l.params;
    accesses("reads", l.reads);
    accesses("writes", l.writes);
    os << "\n";
  }
  // where the activations with memory of their own lie
  for (const auto &a : activationPlan)
    os << "activation name=" << a.name << " id=" << a.id << " offset=" << a.offset
       << " bytes=" << a.bytes << "\n";
  return os.str();
}

} // namespace glow_mi355x
