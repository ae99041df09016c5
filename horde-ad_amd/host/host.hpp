// Host layer above the C ABI of include/hordead_gpu.h: the `Gpu` carrier and
// its tensor-class operations, named after the methods of horde-ad's
// `BaseTensor` class (src/HordeAd/Core/Ops.hs:297-1255) whose `Concrete`
// instance (src/HordeAd/Core/OpsConcrete.hs:97-775) they stand beside.
//
// The layer is written against the table `hgpu_api`, never against a concrete
// library, so the same object code drives the gfx950 library in production and
// any other provider of the ABI a test hands in.
#pragma once
#include <algorithm>
#include <cstdint>
#include <initializer_list>
#include <iterator>
#include <functional>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "hordead_gpu.h"

namespace hordead {

// A shape, or the strides that go with one: a vector of a few extents that sits in
// place up to kInPlace of them (no allocation: shapes are made, copied and dropped
// at every operation) and on the heap beyond.  The part of std::vector's interface
// that the layer uses.
class Shape {
 public:
  using value_type = int64_t;
  using iterator = int64_t*;
  using const_iterator = const int64_t*;
  static constexpr size_t kInPlace = 8;
  Shape() {}
  explicit Shape(size_t n, int64_t v = 0) { grow(n); n_ = n; std::fill(p_, p_ + n, v); }
  Shape(std::initializer_list<int64_t> l) { grow(l.size()); n_ = l.size(); std::copy(l.begin(), l.end(), p_); }
  template <typename It, typename = typename std::iterator_traits<It>::iterator_category>
  Shape(It a, It b) { const size_t n = (size_t)std::distance(a, b); grow(n); n_ = n; std::copy(a, b, p_); }
  Shape(const Shape& o) { grow(o.n_); n_ = o.n_; std::copy(o.p_, o.p_ + n_, p_); }
  Shape(Shape&& o) noexcept { steal(o); }
  Shape(const std::vector<int64_t>& v) : Shape(v.begin(), v.end()) {}
  ~Shape() { if (p_ != in_) delete[] p_; }
  Shape& operator=(const Shape& o) {
    if (this != &o) { n_ = 0; grow(o.n_); n_ = o.n_; std::copy(o.p_, o.p_ + n_, p_); }
    return *this;
  }
  Shape& operator=(Shape&& o) noexcept {
    if (this != &o) { if (p_ != in_) delete[] p_; p_ = in_; cap_ = kInPlace; steal(o); }
    return *this;
  }
  size_t size() const { return n_; }
  bool empty() const { return n_ == 0; }
  int64_t* data() { return p_; }
  const int64_t* data() const { return p_; }
  iterator begin() { return p_; }
  iterator end() { return p_ + n_; }
  const_iterator begin() const { return p_; }
  const_iterator end() const { return p_ + n_; }
  std::reverse_iterator<iterator> rbegin() { return std::reverse_iterator<iterator>(end()); }
  std::reverse_iterator<iterator> rend() { return std::reverse_iterator<iterator>(begin()); }
  std::reverse_iterator<const_iterator> rbegin() const { return std::reverse_iterator<const_iterator>(end()); }
  std::reverse_iterator<const_iterator> rend() const { return std::reverse_iterator<const_iterator>(begin()); }
  int64_t& operator[](size_t i) { return p_[i]; }
  const int64_t& operator[](size_t i) const { return p_[i]; }
  int64_t& at(size_t i) { if (i >= n_) throw std::out_of_range("Shape::at"); return p_[i]; }
  const int64_t& at(size_t i) const { if (i >= n_) throw std::out_of_range("Shape::at"); return p_[i]; }
  int64_t& front() { return p_[0]; }
  const int64_t& front() const { return p_[0]; }
  int64_t& back() { return p_[n_ - 1]; }
  const int64_t& back() const { return p_[n_ - 1]; }
  void clear() { n_ = 0; }
  void reserve(size_t n) { grow(n); }
  void push_back(int64_t v) { grow(n_ + 1); p_[n_++] = v; }
  void emplace_back(int64_t v) { push_back(v); }
  void pop_back() { --n_; }
  void resize(size_t n, int64_t v = 0) { grow(n); if (n > n_) std::fill(p_ + n_, p_ + n, v); n_ = n; }
  void assign(size_t n, int64_t v) { n_ = 0; grow(n); n_ = n; std::fill(p_, p_ + n, v); }
  template <typename It, typename = typename std::iterator_traits<It>::iterator_category>
  void assign(It a, It b) { Shape t(a, b); *this = std::move(t); }
  iterator insert(const_iterator at, int64_t v) { return insert(at, &v, &v + 1); }
  template <typename It, typename = typename std::iterator_traits<It>::iterator_category>
  iterator insert(const_iterator at, It a, It b) {
    const size_t i = (size_t)(at - p_), k = (size_t)std::distance(a, b);
    if (k == 0) return p_ + i;
    int64_t tmp_in[kInPlace];   // the range may lie in this very object
    std::vector<int64_t> tmp_big;
    int64_t* src = tmp_in;
    if (k > kInPlace) { tmp_big.assign(a, b); src = tmp_big.data(); } else std::copy(a, b, tmp_in);
    grow(n_ + k);
    std::copy_backward(p_ + i, p_ + n_, p_ + n_ + k);
    std::copy(src, src + k, p_ + i);
    n_ += k;
    return p_ + i;
  }
  iterator erase(const_iterator at) { return erase(at, at + 1); }
  iterator erase(const_iterator a, const_iterator b) {
    const size_t i = (size_t)(a - p_), j = (size_t)(b - p_);
    std::copy(p_ + j, p_ + n_, p_ + i);
    n_ -= j - i;
    return p_ + i;
  }
  void swap(Shape& o) { Shape t(std::move(o)); o = std::move(*this); *this = std::move(t); }
  friend bool operator==(const Shape& a, const Shape& b) { return a.n_ == b.n_ && std::equal(a.p_, a.p_ + a.n_, b.p_); }
  friend bool operator!=(const Shape& a, const Shape& b) { return !(a == b); }
  friend bool operator<(const Shape& a, const Shape& b) { return std::lexicographical_compare(a.begin(), a.end(), b.begin(), b.end()); }
  operator std::vector<int64_t>() const { return std::vector<int64_t>(begin(), end()); }

 private:
  void grow(size_t n) {
    if (n <= cap_) return;
    size_t c = cap_ * 2 > n ? cap_ * 2 : n;
    int64_t* q = new int64_t[c];
    std::copy(p_, p_ + n_, q);
    if (p_ != in_) delete[] p_;
    p_ = q;
    cap_ = c;
  }
  void steal(Shape& o) {
    n_ = o.n_;
    if (o.p_ == o.in_) { std::copy(o.in_, o.in_ + n_, in_); }
    else { p_ = o.p_; cap_ = o.cap_; o.p_ = o.in_; o.cap_ = kInPlace; }
    o.n_ = 0;
  }
  int64_t in_[kInPlace];
  int64_t* p_ = in_;
  size_t n_ = 0, cap_ = kInPlace;
};

struct HostError : std::runtime_error {
  int code;
  HostError(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};

class T;
struct ArrHolder;

// One provider of the array ABI plus a context on it.
struct Backend {
  const hgpu_api* api;
  hgpu_ctx* ctx;
  std::map<std::pair<int, int64_t>, std::shared_ptr<ArrHolder>> iota_cache;   // (dtype, n)
  std::map<std::pair<int, uint64_t>, std::shared_ptr<ArrHolder>> const_cache; // (dtype, value bits)
  bool capturing = false;   // between hh_capture_begin and hh_capture_end
  bool fuse = true;   // defer elementwise operations into fused programs (when the provider has fused_map)
  uint64_t walk_gen = 0;    // walks over pending expressions number themselves: a node seen carries the walk's number
  std::vector<std::weak_ptr<ArrHolder>> pending_dimsums;   // sums over all dims but one of an expression, not yet taken (ArrHolder::ones_b)
  std::vector<std::weak_ptr<ArrHolder>> pending_sums;   // sums of all elements of an expression, not yet taken (ArrHolder::ssrc)
  std::map<std::string, int64_t> counters;   // how often each rewrite onto a fused entry point was taken (diagnostic)
  void check(int rc) const;
};

// Shape, element strides and offset of a strided view over the dense row-major
// layout of some value.
struct Meta {
  Shape shape, strides;
  int64_t offset = 0;
};

struct ArrHolder {
  Backend* be;
  hgpu_array* h;
  // Small integer arrays that came from the host keep their values: index
  // functions that look constants up in them can then be folded on the host.
  std::shared_ptr<std::vector<int64_t>> host_i64;
  bool host_i64_folded = false;   // some index function has been simplified with these values: they must not change any more
  // The one-element array this array repeats at every position (set by broadcast_scalar).
  std::shared_ptr<ArrHolder> scalar_src;
  // A pending elementwise product fa * fb (h == nullptr until it is needed as
  // an array).  Views of it stay pending, and summing it is a contraction of
  // the two factors, so `tssumN (u * v)` never writes the product to memory.
  // With keep >= 0 the pending value is instead the CONTRACTION of fa and fb
  // over all but their first `keep` dims (the sum of a pending product): a
  // scatter with an affine index function folds into it (the transposed
  // convolution never writes its patch gradient to memory).
  std::shared_ptr<ArrHolder> fa, fb;
  int keep = -1;
  // The product expression whose factors fa and fb are (tssumN (u * v) taken apart): when somebody has written
  // the product out by the time the contraction is computed, the contraction is the sum of that array.
  std::shared_ptr<ArrHolder> whole;
  // Further (fa, fb) pairs of a pending SUM of contractions of one shape (the
  // cotangent of a parameter used once per step of an unrolled recurrence):
  // written out by one grouped launch when the provider has contract_sum.
  std::vector<std::pair<std::shared_ptr<ArrHolder>, std::shared_ptr<ArrHolder>>> more;
  // fb is all ones: the value is the SUM of fa over its trailing dims.  When fa
  // is a transposed view of an expression (a bias's cotangent: the layer's
  // cotangent summed over batch, height and width) the sum waits for the pass
  // that writes the expression out and is taken in that pass
  // (Backend::pending_dimsums, hgpu_fused_map_dimsum).
  bool ones_b = false;
  uint64_t walk_mark = 0;   // the last walk over pending expressions that has seen this node (Backend::walk_gen)
  // A pending contraction that is a transpose of another pending contraction
  // remembers it: if anyone else still wants the original, the original is
  // computed once and this one becomes a view of it.
  std::shared_ptr<ArrHolder> origin;
  std::vector<int> origin_perm;
  // A pending CONCATENATION along the first dim (h == nullptr, pieces not
  // empty): `tsappend`, and the zero-extension that is the adjoint of a slice
  // (a piece without an array is zeros).  Slicing it hands back the pieces, and
  // adding two of them piece by piece adds only where both have data -- the
  // stacked state of an unrolled recurrence and its cotangent are then never
  // copied, cleared or added as a whole.
  // A pending expression over a REFINED index space (h == nullptr, mv_inner
  // set): mv_inner has the shape of this value with some dims split in two or
  // more (mv_groups[d] adjacent dims of it make dim d of mv_shape).  Written out
  // densely, the inner array IS this value (merging dims of a dense array is
  // free), so elementwise consumers are evaluated over the refined space and
  // `out[2 i + p, 2 j + q] = src[i, j, p, q]` -- the adjoint of taking pooling
  // windows -- costs no pass of its own.
  std::shared_ptr<ArrHolder> mv_inner;
  Shape mv_shape;
  std::vector<int> mv_groups;
  struct Piece { int64_t len; std::shared_ptr<ArrHolder> v; };
  std::vector<Piece> pieces;
  Shape pshape;
  int pdtype = 0;
  // A pending ELEMENTWISE operation (h == nullptr): kind/op as in
  // hgpu_fused_instr, operands fa, fb, fc.  Chains of them are handed to the
  // provider's fused_map as one program when the value is first needed as an
  // array, so that `x * sin y + z` is one pass over memory, not three.
  int ekind = -1, eop = 0, edtype = 0;
  std::shared_ptr<ArrHolder> fc;
  int esize = 0;          // pending nodes beneath, to bound program size
  Shape eshape;
  // The result of tsargMin / tsargMax over the last dim remembers its source and
  // the extremal values the same pass produced: `sindex0 t [kargMin t]` (the
  // minimum of the reference's soft-max loss) is then those values, not a gather.
  std::shared_ptr<ArrHolder> arg_src, arg_values;
  // A pending VIEW (h == nullptr, ekind < 0, vsrc set): the strided view vmeta
  // over the dense row-major (and possibly zero-extended, vlo / vhi) result of vsrc, a value that is itself still
  // pending (a contraction, an elementwise expression).  Views of it compose
  // on the host; it is computed by computing vsrc once and viewing that.  An
  // elementwise expression made by viewing the leaves of another one (ekind >= 0)
  // carries the same two fields as a note: it equals that view of vsrc's result.
  std::shared_ptr<ArrHolder> vsrc;
  Meta vmeta;
  // ... of vsrc's result zero-extended by vlo / vhi per dim (empty: not extended)
  Shape vlo, vhi;
  // A pending SUM (h == nullptr, ssrc set): the sum of all elements of the
  // pending expression ssrc.  It is taken in the pass that writes other
  // expressions of the same shape out (an objective's value in the pass of its
  // gradient), or by a pass of its own when somebody needs it first.
  std::shared_ptr<ArrHolder> ssrc;
  // A stand-in without data that view operations are tried on to learn the
  // strides they produce (vmeta holds its shape and strides).
  bool probe = false;
  int probe_dtype = 0;
  ArrHolder(Backend* b, hgpu_array* a) : be(b), h(a) {}
  ~ArrHolder() { if (h) be->api->release(h); }
  ArrHolder(const ArrHolder&) = delete;
  void force();
  bool view_of_written_source();
};

// Memory for the holders: a training step makes thousands of them and frees most together when its
// tape goes, more than the allocator's per-thread cache of one block size holds, so freed blocks are
// kept on a list per thread (and per block size) and handed out again.
template <size_t N>
struct BlockList {
  struct Node { Node* next; };
  Node* head = nullptr;
  size_t n = 0;
  ~BlockList() {
    while (head) { Node* x = head; head = head->next; ::operator delete(x); }
  }
  static BlockList& mine() {
    static thread_local BlockList l;
    return l;
  }
};
template <typename U>
struct BlockAlloc {
  using value_type = U;
  BlockAlloc() = default;
  template <typename V> BlockAlloc(const BlockAlloc<V>&) {}
  U* allocate(size_t k) {
    if (k == 1) {
      auto& l = BlockList<sizeof(U)>::mine();
      if (l.head) {
        auto* x = l.head;
        l.head = x->next;
        --l.n;
        return reinterpret_cast<U*>(x);
      }
    }
    return static_cast<U*>(::operator new(k * sizeof(U)));
  }
  void deallocate(U* p, size_t k) {
    auto& l = BlockList<sizeof(U)>::mine();
    if (k != 1 || l.n >= 16384) { ::operator delete(p); return; }
    auto* x = reinterpret_cast<typename BlockList<sizeof(U)>::Node*>(p);
    x->next = l.head;
    l.head = x;
    ++l.n;
  }
  template <typename V> bool operator==(const BlockAlloc<V>&) const { return true; }
  template <typename V> bool operator!=(const BlockAlloc<V>&) const { return false; }
};
inline std::shared_ptr<ArrHolder> new_holder(Backend* be, hgpu_array* h) { return std::allocate_shared<ArrHolder>(BlockAlloc<ArrHolder>(), be, h); }

// `Gpu (TKS sh r)`: an immutable strided view on the device.  Scalars
// (`TKScalar r`) are rank-0 views, so that they never force a device sync.
class T {
 public:
  T() {}
  T(Backend* be, hgpu_array* h) : p_(new_holder(be, h)) {}
  explicit T(std::shared_ptr<ArrHolder> p) : p_(std::move(p)) {}
  const std::shared_ptr<ArrHolder>& holder() const { return p_; }
  bool valid() const { return (bool)p_; }
  Backend* be() const { return p_->be; }
  hgpu_array* h() const {
    if (!p_->h) p_->force();
    return p_->h;
  }
  bool pending_expr() const { return p_ && !p_->h && p_->ekind >= 0; }
  bool is_probe() const { return p_ && p_->probe; }
  bool pending_sum() const { return p_ && !p_->h && p_->ssrc; }
  bool pending_view() const { return p_ && !p_->h && p_->ekind < 0 && p_->vsrc && !p_->probe; }
  bool meta_only() const { return is_probe() || pending_view(); }   // shape and strides known on the host, no array yet
  bool pending_product() const { return pending_expr() && p_->ekind == HGPU_FUSED_OP2 && p_->eop == HGPU_MUL; }
  bool pending_pieces() const { return p_ && !p_->h && !p_->pieces.empty(); }
  bool pending_merged() const { return p_ && !p_->h && p_->mv_inner; }
  bool contraction_like() const { return p_ && !p_->h && p_->ekind < 0 && p_->fa && p_->keep >= 0; }
  bool pending_contraction() const { return contraction_like() && p_->more.empty(); }   // a single one: open to rewrites
  int pending_keep() const { return p_->keep; }
  T factor_a() const { return T(p_->fa); }
  T factor_b() const { return T(p_->fb); }
  // metadata never forces a pending product: the first factor has the same
  hgpu_array* meta_h() const {
    const ArrHolder* q = p_.get();
    while (!q->h && q->fa) q = q->fa.get();
    return q->h;
  }
  int rank() const {
    if (pending_sum()) return 0;
    if (meta_only()) return (int)p_->vmeta.shape.size();
    if (pending_pieces()) return (int)p_->pshape.size();
    if (pending_merged()) return (int)p_->mv_shape.size();
    if (pending_expr()) return (int)p_->eshape.size();
    return contraction_like() ? p_->keep : be()->api->rank(meta_h());
  }
  int dtype() const {
    if (pending_sum()) return T(p_->ssrc).dtype();
    if (is_probe()) return p_->probe_dtype;
    if (pending_view()) return T(p_->vsrc).dtype();
    if (pending_pieces()) return p_->pdtype;
    if (pending_merged()) return T(p_->mv_inner).dtype();
    return pending_expr() ? p_->edtype : T(p_->fa ? p_->fa : p_).dtype_of_holder();
  }
  int dtype_of_holder() const { return p_->h ? be()->api->dtype_of(p_->h) : dtype(); }
  int64_t size() const {
    int64_t n = 1;
    for (auto e : shape()) n *= e;
    return n;
  }
  Shape shape() const;
  Shape strides() const;
  const std::shared_ptr<std::vector<int64_t>>& host_i64() const { return p_->host_i64; }
  void set_host_i64(std::shared_ptr<std::vector<int64_t>> v) { p_->host_i64 = std::move(v); }

 private:
  std::shared_ptr<ArrHolder> p_;
};

// ---- array primitives (one ABI call each) ---------------------------------
T upload(Backend* be, int dtype, const Shape& shape, const void* host);
T constant(Backend* be, int dtype, double value);                 // cached rank-0 array
T constant_i(Backend* be, int dtype, int64_t value);
T iota(Backend* be, int64_t n, int dtype);                         // cached
T transpose(const T& a, const std::vector<int>& perm);
T reshape(const T& a, const Shape& shape);
T slice(const T& a, int dim, int64_t start, int64_t len);
T reverse(const T& a, int dim);
T replicate(const T& a, const Shape& prefix);
T index_prefix(const T& a, const Shape& ix);
T as_strided(const T& a, const Shape& shape, const Shape& strides, int64_t offset);
T materialize(const T& a);
T pad(const T& a, const Shape& lo, const Shape& hi);
T ewise1(int op, const T& a);
T ewise2(int op, const T& a, const T& b);
T lazy_mul(const T& a, const T& b);                                // a * b, not yet written to memory
void force_many(const std::vector<T>& ts);                         // pending values of one shape share a pass
T lazy_contract(const T& a, const T& b, int n_keep);               // sum of a * b over the trailing dims, pending
T add_cotangents(const T& a, const T& b);                          // a + b; pending contractions of one shape stay a pending sum
T compare(int cmp, const T& a, const T& b);
bool compare_all(int cmp, const T& a, const T& b);
T select(const T& c, const T& a, const T& b);
T convert(const T& a, int dtype, int mode);
T contract(const T& a, const T* b, int n_keep);
T argminmax_last(const T& a, bool want_max);
T concat(const std::vector<T>& parts);
T gather_raw(const T& src, const std::vector<T>& ix, const Shape& shm);
T scatter_raw(const T& src, const std::vector<T>& ix, int rank_m, const Shape& shp, int flags);
T onehot(const T& v, const Shape& ix, const Shape& shp);
T zeros(Backend* be, int dtype, const Shape& shape);               // stride-0 view of a cached 0
// optimizer.cpp (External/OptimizerTools.hs)
T update_with_gradient(double gamma, const T& p, const T& g);
void adam_update(const T& alphat, double beta1, double beta2, double epsilon, const T& m, const T& v, const T& p, const T& g, T* m_new, T* v_new, T* p_new);
T adam_step_size(Backend* be, int dtype, double alpha, double beta1, double beta2, int t_new);
void assign(const T& dst, const T& src);                           // dst's memory takes src's elements
T broadcast_scalar(const T& s, const Shape& shape);                // tsreplicate0N

// ---- BaseTensor-named operations (Ops.hs line of each method in the .cpp) --
T tssum(const T& t);                       // sum over the outermost dim
T tssumN(const T& t, int k);               // sum over the k outermost dims
T tssum0(const T& t);
T tsdot0(const T& a, const T& b);
T tsdot1In(const T& a, const T& b);        // contraction over the innermost dim
T tsdotNIn(const T& a, const T& b, int n); // contraction over the n innermost dims
T tsmatvecmul(const T& m, const T& v);
T tsmatmul2(const T& m1, const T& m2);
T tsreplicate(const T& t, int64_t k);
T tsreplicateN(const T& t, const Shape& shm);
T tsreplicate0N(const T& scalar, const Shape& sh);
T tsappend(const T& a, const T& b);
T tsslice(const T& t, int64_t i, int64_t n);
T tsreverse(const T& t);
T tstranspose(const T& t, const std::vector<int>& perm);
T tsreshape(const T& t, const Shape& sh);
T tsindex(const T& t, const Shape& ix);    // concrete (host) indices
T tsoneHot(const T& v, const Shape& ix, const Shape& shp);
T tsfloor(const T& t, int dtype);
T tsfromIntegral(const T& t, int dtype);
T tscast(const T& t, int dtype);
T tsargMin(const T& t);
T tsargMax(const T& t);
T tsiota(Backend* be, int64_t n, int dtype);

// ---- lane-batched scalars: the `IntOf Gpu` an index function is applied to --
//
// horde-ad hands gather/scatter/build an index FUNCTION over scalars
// (Ops.hs:689-705); `Concrete` calls it once per position
// (OpsConcrete.hs:1581-1665).  Here the function is called ONCE with symbolic
// position variables; every scalar it computes is an `Ix`: a value for all
// positions of the space `shm` at a time -- an affine form in the position
// variables when that is provable (then gathers become strided views), or a
// device array of shape shm otherwise.
struct Ix {
  Shape shm;                   // the position space this value ranges over
  bool affine = false;
  int64_t c0 = 0;              // affine: c0 + sum_d coef[d] * m_d
  std::vector<int64_t> coef;
  T arr;                       // otherwise: array of shape shm (any dtype, any strides)
  int dtype = HGPU_I64;
  // kargMin / kargMax of `arg_of !$ [m_0, ..]` at the position itself: the
  // extremal values came out of the same pass (arg_vals), so a gather of
  // arg_of at [m_0, .., this] is arg_vals.
  std::shared_ptr<ArrHolder> arg_of;
  T arg_vals;
  // ifH cond a b with constant a, b: a gather from a table by this index alone is
  // a choice between two of the table's elements (`sgather [0.0, 1.0] (\.. -> [ifH c 0 1])`,
  // the mask of relu in the reference's simplified programs, test/simplified/TestMnistPP.hs:735).
  T sel_cond;
  int64_t sel_a = 0, sel_b = 0;
};

Ix ix_var(Backend* be, const Shape& shm, int d);
Ix ix_const(Backend* be, const Shape& shm, int dtype, double v);
Ix ix_lift(const Shape& shm, const T& scalar);            // a rank-0 tensor seen from every position
T ix_array(Backend* be, const Ix& x);                     // as a device array of shape shm
Ix ix_op1(Backend* be, int op, const Ix& a);
Ix ix_op2(Backend* be, int op, const Ix& a, const Ix& b);
Ix ix_compare(Backend* be, int cmp, const Ix& a, const Ix& b);
Ix ix_select(Backend* be, const Ix& c, const Ix& a, const Ix& b);   // kcond / ifH
Ix ix_convert(Backend* be, const Ix& a, int dtype, int mode);
Ix ix_index0(Backend* be, const T& t, const std::vector<Ix>& ix);   // tsindex0 at batched indices
// kargMin / kargMax (t !$ ix): arg-extremum of the last dim of the batched partial index
Ix ix_argminmax(Backend* be, const T& t, const std::vector<Ix>& ix, bool want_max);

// tsgather (Ops.hs:701-705) / tsscatter (Ops.hs:689-693) with the index
// function already applied to the symbolic positions.
T tsgather(const T& src, const Shape& shm, const std::vector<Ix>& ix);
T tsscatter(const T& src, int rank_m, const Shape& shp, const std::vector<Ix>& ix);

// ---- dual numbers: reverse-mode differentiation over the carrier -----------
//
// Mirror of `ADVal target` + `gradientFromDelta` (OpsADVal.hs:44-60,
// DeltaEval.hs:64-78,391-595) for the operations above: every operation on a
// `D` runs the primal operation on the carrier and records the transposition
// rule; `backward` plays the records in reverse.
struct Tape;
struct D {
  T primal;
  int node = -1;               // index into the tape; -1 = no derivative flows
};

struct Tape {
  struct Rec {
    std::function<void(const T& cot, std::vector<T>& slots)> back;
  };
  Backend* be;
  std::vector<Rec> recs;
  explicit Tape(Backend* b) : be(b) {}
  D input(const T& t);                                     // differentiable leaf
  int push(std::function<void(const T&, std::vector<T>&)> f);
  // Cotangents of `inputs` given d(out) = dt.
  std::vector<T> backward(const D& out, const T& dt, const std::vector<D>& inputs);
};

D d_const(const T& t);
D d_ewise1(Tape& tp, int op, const D& a);
D d_ewise2(Tape& tp, int op, const D& a, const D& b);
D d_select(Tape& tp, const T& cond, const D& a, const D& b);
D d_convert(Tape& tp, const D& a, int dtype, int mode);
D d_tssumN(Tape& tp, const D& t, int k);
D d_tssum0(Tape& tp, const D& t);
D d_tsdot0(Tape& tp, const D& a, const D& b);
D d_tsdot1In(Tape& tp, const D& a, const D& b);
D d_tsdotNIn(Tape& tp, const D& a, const D& b, int n);
D d_tD(const D& primal, const D& dual);                 // tD: primal part of one, dual part of the other
D d_tsmatmul2(Tape& tp, const D& a, const D& b);
D d_tsreplicateN(Tape& tp, const D& t, const Shape& shm);
D d_tsappend(Tape& tp, const D& a, const D& b);
D d_tsslice(Tape& tp, const D& t, int64_t i, int64_t n);
D d_tsreverse(Tape& tp, const D& t);
D d_tstranspose(Tape& tp, const D& t, const std::vector<int>& perm);
D d_tsreshape(Tape& tp, const D& t, const Shape& sh);
D d_tsindex(Tape& tp, const D& t, const Shape& ix);
D d_tsgather(Tape& tp, const D& src, const Shape& shm, const std::vector<Ix>& ix);
D d_tsscatter(Tape& tp, const D& src, int rank_m, const Shape& shp, const std::vector<Ix>& ix);

}  // namespace hordead
