// Thin PyTorch C++ binding of the C ABI (include/managan_hip.h) for the operators that the reference exposes from its
// three compiled extensions, with the reference's signatures:
//   neighbour_grid_cuda   get_edges, get_neighbours, edges_read, edges_reduce
//                         (extensions/neighbour_grid/neighbour_grid.cpp:59-203)
//   tensor_ops_cuda       tensor_linear, differentiable (extensions/tensor_ops/tensor_ops.cpp:31-182)
//   codegen_tensops_cuda  bee_fwd / bee_bwl / bee_bwr, cow_o0 / cow_o1 fwd / bwl / bwr
//                         (extensions/codegen_tensops/codegen_tensops.cpp:1519-1978)
// Every function validates like the reference's front end (same messages), allocates its outputs with torch on the
// inputs' device, and enqueues on torch's current stream of that device.  No arithmetic happens here: the kernels are
// in libmanagan_hip.so.  Host C++ only (compiled with the host compiler: no device code, no GPU runtime calls of its
// own), so that a call costs a few microseconds of host time where the ctypes route costs about twelve.
#include <torch/extension.h>
// torch's ROCm build presents its devices under the device type "cuda": the guard and stream types that know this
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <array>
#include <cstdint>
#include <string>
#include <tuple>
#include <vector>

#include "managan_hip.h"

namespace {

constexpr const char* kBeeOrder[13] = {"000", "110", "220", "011", "101", "121", "211",
                                       "022", "202", "112", "222", "111", "212"};

void check_input(const at::Tensor& t, const char* name, at::ScalarType dtype = at::kFloat) {
    TORCH_CHECK(t.is_cuda(), name, " must be a CUDA tensor");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(t.scalar_type() == dtype, "expected scalar type ", c10::toString(dtype), " but found ",
                c10::toString(t.scalar_type()), " for ", name);
}

// a non-zero status as the exception the reference would raise (the same texts as the ctypes route)
void check(int status) {
    if (status == MG_OK) return;
    TORCH_CHECK(status != MG_ERR_BOX_TOO_SMALL, "box dimension must be greater than 3*cutoff");
    const char* text = mg_last_error();
    TORCH_CHECK(false, mg_status_string(status), text[0] ? ": " : "", text);
}

mg_stream_t stream_of(const at::Tensor& t) {
    return reinterpret_cast<mg_stream_t>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream());
}

const float* fp(const at::Tensor& t) { return t.data_ptr<float>(); }
float* fp(at::Tensor& t) { return t.data_ptr<float>(); }

std::vector<int64_t> shape_of(int64_t rows, int64_t chan, int rank) {
    std::vector<int64_t> s{rows, chan};
    for (int k = 0; k < rank; k++) s.push_back(3);
    return s;
}

// exactly (R,C), (R,C,3), (R,C,3,3) with common R and C
std::pair<int64_t, int64_t> rows_chan(std::initializer_list<const at::Tensor*> by_rank,
                                      std::initializer_list<const char*> names) {
    int64_t rows = -1, chan = -1;
    int rank = 0;
    auto name = names.begin();
    for (const at::Tensor* t : by_rank) {
        check_input(*t, *name);
        TORCH_CHECK(t->dim() == 2 + rank, *name, " has wrong number of axes");
        for (int ax = 0; ax < rank; ax++) TORCH_CHECK(t->size(2 + ax) == 3, *name, " must have size 3 on tensor axes");
        if (rows < 0) { rows = t->size(0); chan = t->size(1); }
        TORCH_CHECK(t->size(0) == rows, *name, " batch size mismatch");
        TORCH_CHECK(t->size(1) == chan, *name, " channel size mismatch");
        ++rank;
        ++name;
    }
    return {rows, chan};
}

// ------------------------------------------------------------------ neighbour_grid_cuda
struct Search {
    at::Tensor workspace, row_ptr, edge_counts;
    int stats[4];
};

// count phase + read-back of the four statistics (the reference's front end also synchronises to size its outputs)
Search count_phase(float cutoff, float bx, float by, float bz, const at::Tensor& x) {
    check_input(x, "x");
    TORCH_CHECK(x.dim() == 3 && x.size(2) == 3, "x must have shape (batch, nodes, 3)");
    const int batch = (int)x.size(0), nodes = (int)x.size(1);
    size_t bytes = 0;
    check(mg_neighbour_workspace_bytes(batch, nodes, cutoff, bx, by, bz, &bytes));
    const auto i32 = x.options().dtype(at::kInt);
    Search s;
    s.workspace = torch::empty({(int64_t)bytes}, x.options().dtype(at::kByte));
    s.row_ptr = torch::empty({(int64_t)batch * nodes + 1}, i32);
    s.edge_counts = torch::empty({batch}, i32);
    at::Tensor stats = torch::empty({4}, i32);
    check(mg_neighbour_count(fp(x), batch, nodes, cutoff, bx, by, bz, s.workspace.data_ptr(), bytes,
                             s.row_ptr.data_ptr<int>(), s.edge_counts.data_ptr<int>(), stats.data_ptr<int>(),
                             stream_of(x)));
    const at::Tensor host = stats.cpu();
    for (int k = 0; k < 4; k++) s.stats[k] = host.data_ptr<int>()[k];
    TORCH_CHECK((s.stats[3] & 1) == 0, "edge count does not fit int32");
    return s;
}

// the reference's overflow errors, in the reference's order (neighbour_grid_kern.cu:195-217)
void check_caps(const Search& s, int listmax, int neighboursmax) {
    TORCH_CHECK(s.stats[1] <= listmax, "Cell list overflow occurred. Trying increasing listmax.");
    TORCH_CHECK(listmax == 32 || listmax == 64 || listmax == 128 || listmax == 256,
                "expected listmax to be one of 32, 64, 128, 256. other values not supported!");
    TORCH_CHECK(s.stats[2] <= neighboursmax, "Neighbour list overflow occurred. Try increasing neighboursmax.");
}

std::pair<at::Tensor, at::Tensor> fill_phase(const Search& s, float cutoff, float bx, float by, float bz,
                                             const at::Tensor& x) {
    const auto i32 = x.options().dtype(at::kInt);
    at::Tensor src = torch::empty({s.stats[0]}, i32), dst = torch::empty({s.stats[0]}, i32);
    check(mg_neighbour_fill(s.workspace.data_ptr(), (size_t)s.workspace.numel(), (int)x.size(0), (int)x.size(1), cutoff, bx,
                            by, bz, s.row_ptr.data_ptr<int>(), s.stats[0], src.data_ptr<int>(), dst.data_ptr<int>(),
                            stream_of(x)));
    return {src, dst};
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> get_edges(int listmax, int neighboursmax, float cutoff, float bx, float by,
                                                         float bz, const at::Tensor& x) {
    check_input(x, "x");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    const Search s = count_phase(cutoff, bx, by, bz, x);
    check_caps(s, listmax, neighboursmax);
    auto edges = fill_phase(s, cutoff, bx, by, bz, x);
    return {edges.first, edges.second, s.edge_counts};
}

std::tuple<at::Tensor, at::Tensor> get_neighbours(int listmax, int neighboursmax, float cutoff, float bx, float by,
                                                  float bz, const at::Tensor& x) {
    check_input(x, "x");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    const Search s = count_phase(cutoff, bx, by, bz, x);
    check_caps(s, listmax, neighboursmax);
    auto edges = fill_phase(s, cutoff, bx, by, bz, x);
    const int batch = (int)x.size(0), nodes = (int)x.size(1);
    const auto i32 = x.options().dtype(at::kInt);
    at::Tensor neighbours = torch::empty({batch, nodes, neighboursmax}, i32), counts = torch::empty({batch, nodes}, i32);
    check(mg_neighbour_pad(s.row_ptr.data_ptr<int>(), edges.second.data_ptr<int>(), batch, nodes, neighboursmax,
                           neighbours.data_ptr<int>(), counts.data_ptr<int>(), stream_of(x)));
    return {neighbours, counts};
}

at::Tensor edges_read(const at::Tensor& counts, const at::Tensor& neighbours, const at::Tensor& x) {
    check_input(counts, "neighbourCounts", at::kInt);
    check_input(neighbours, "neighbours", at::kInt);
    check_input(x, "x");
    TORCH_CHECK(counts.dim() == 2, "neighbourCounts must have shape (batch, nodes)");
    TORCH_CHECK(neighbours.dim() == 3, "neighbourCounts must have shape (batch, nodes, neighboursmax)");
    TORCH_CHECK(x.dim() == 3, "x must have shape (batch, nodes, chan)");
    const int64_t B = counts.size(0), N = counts.size(1);
    TORCH_CHECK(B == neighbours.size(0) && B == x.size(0), "batch dimension of all tensors must match");
    TORCH_CHECK(N == neighbours.size(1) && N == x.size(1), "node dimension of all tensors must match");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    const int nmax = (int)neighbours.size(2), chan = (int)x.size(2);
    at::Tensor out = torch::empty({B, N, nmax, chan}, x.options());
    check(mg_padded_edges_read(counts.data_ptr<int>(), neighbours.data_ptr<int>(), fp(x), (int)B, (int)N, nmax, chan, fp(out),
                               stream_of(x)));
    return out;
}

at::Tensor edges_reduce(const at::Tensor& counts, const at::Tensor& neighbours, const at::Tensor& x) {
    check_input(counts, "neighbourCounts", at::kInt);
    check_input(neighbours, "neighbours", at::kInt);
    check_input(x, "x");
    TORCH_CHECK(counts.dim() == 2, "neighbourCounts must have shape (batch, nodes)");
    TORCH_CHECK(neighbours.dim() == 3, "neighbours must have shape (batch, nodes, neighboursmax)");
    TORCH_CHECK(x.dim() == 4, "x must have shape (batch, nodes, neighboursmax, chan)");
    const int64_t B = counts.size(0), N = counts.size(1);
    TORCH_CHECK(B == neighbours.size(0) && B == x.size(0), "batch dimension of all tensors must match");
    TORCH_CHECK(N == neighbours.size(1) && N == x.size(1), "node dimension of all tensors must match");
    TORCH_CHECK(neighbours.size(2) == x.size(2), "neighboursmax dimension must match between neighbours and x");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    const int nmax = (int)neighbours.size(2), chan = (int)x.size(3);
    at::Tensor out = torch::empty({B, N, chan}, x.options());
    check(mg_padded_edges_reduce(counts.data_ptr<int>(), fp(x), (int)B, (int)N, nmax, chan, fp(out), stream_of(x)));
    return out;
}

// ------------------------------------------------------------------ tensor_ops_cuda
struct LinearDims {
    int64_t rows, dim_in, dim_out;
    std::vector<int64_t> y_shape;
};

LinearDims linear_dims(int64_t inds, const at::Tensor& W, const at::Tensor& x) {
    TORCH_CHECK(W.is_cuda(), "W must be a CUDA tensor");
    TORCH_CHECK(W.scalar_type() == at::kFloat, "expected scalar type Float but found ", c10::toString(W.scalar_type()),
                " for W");
    check_input(x, "x");
    TORCH_CHECK(W.dim() == 2, "expected W to be a matrix (2 dims)");
    TORCH_CHECK(inds >= 0 && inds <= 2, "tensor_linear currently only supports a number of indices up to 2.");
    LinearDims d;
    d.dim_out = W.size(0);
    d.dim_in = W.size(1);
    d.y_shape = x.sizes().vec();
    const int64_t batch_dims = (int64_t)d.y_shape.size() - (1 + inds);
    TORCH_CHECK(batch_dims >= 0, "x has too few dims");
    TORCH_CHECK(d.y_shape[batch_dims] == d.dim_in, "channel dim size mismatch for x");
    for (int64_t i = batch_dims + inds; i > batch_dims; i--)
        TORCH_CHECK(d.y_shape[i] == 3, "expected tensor index dim to be 3d for input x");
    d.rows = 1;
    for (int64_t i = 0; i < batch_dims; i++) d.rows *= d.y_shape[i];
    d.y_shape[batch_dims] = d.dim_out;
    return d;
}

// y[..., o, t] = sum_i W[o, i] x[..., i, t]; W is read through its strides (a transposed view costs nothing)
at::Tensor linear_forward(int64_t inds, const at::Tensor& W, const at::Tensor& x) {
    const LinearDims d = linear_dims(inds, W, x);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    at::Tensor y = torch::empty(d.y_shape, x.options());
    if (d.rows == 0 || d.dim_out == 0) return y;
    if (d.dim_in == 0) return y.zero_();
    check(mg_tensor_linear((int)inds, fp(W), W.stride(0), W.stride(1), fp(x), d.rows, (int)d.dim_in, (int)d.dim_out, nullptr,
                           0, 0, fp(y), stream_of(x)));
    return y;
}

// dW[o, i] = sum over rows and components of dy[r, o, t] x[r, i, t]
at::Tensor linear_weight_grad(int64_t inds, const at::Tensor& dy, const at::Tensor& x, int64_t dim_out, int64_t dim_in) {
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
    int64_t T = 1;
    for (int64_t k = 0; k < inds; k++) T *= 3;
    const int64_t rows = dim_in > 0 ? x.numel() / (dim_in * T) : 0;
    at::Tensor dW = torch::empty({dim_out, dim_in}, x.options());
    if (dW.numel() == 0) return dW;
    if (rows == 0) return dW.zero_();
    size_t bytes = 0;
    check(mg_tensor_linear_wgrad_workspace_bytes(rows, (int)dim_in, (int)dim_out, &bytes));
    at::Tensor ws = torch::empty({(int64_t)bytes}, x.options().dtype(at::kByte));
    check(mg_tensor_linear_wgrad((int)inds, fp(dy), fp(x), rows, (int)dim_in, (int)dim_out, ws.data_ptr(), fp(dW),
                                 stream_of(x)));
    return dW;
}

// The forward, the input gradient (the same contraction with the transposed view of W) and the weight gradient are
// each other's derivatives, so the function differentiates to any order (the reference's stops after the first).
struct WeightGradFn;

struct TensorLinearFn : public torch::autograd::Function<TensorLinearFn> {
    static at::Tensor forward(torch::autograd::AutogradContext* ctx, int64_t inds, const at::Tensor& W, const at::Tensor& x) {
        ctx->saved_data["inds"] = inds;
        ctx->save_for_backward({W, x});
        return linear_forward(inds, W, x);
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                   torch::autograd::variable_list grads);
};

struct WeightGradFn : public torch::autograd::Function<WeightGradFn> {
    static at::Tensor forward(torch::autograd::AutogradContext* ctx, int64_t inds, const at::Tensor& dy, const at::Tensor& x,
                              int64_t dim_out, int64_t dim_in) {
        ctx->saved_data["inds"] = inds;
        ctx->save_for_backward({dy, x});
        return linear_weight_grad(inds, dy.contiguous(), x, dim_out, dim_in);
    }
    static torch::autograd::variable_list backward(torch::autograd::AutogradContext* ctx,
                                                   torch::autograd::variable_list grads) {
        const auto saved = ctx->get_saved_variables();
        const int64_t inds = ctx->saved_data["inds"].toInt();
        const at::Tensor &dy = saved[0], &x = saved[1];
        const at::Tensor g = grads[0].contiguous();                   // (dim_out, dim_in)
        at::Tensor d_dy, d_x;
        // (needs_input_grad counts the tensor arguments only: dy is 0, x is 1)
        if (ctx->needs_input_grad(0)) d_dy = TensorLinearFn::apply(inds, g, x);                       // g x
        if (ctx->needs_input_grad(1)) d_x = TensorLinearFn::apply(inds, g.t(), dy.contiguous());      // g^T dy
        return {at::Tensor(), d_dy, d_x, at::Tensor(), at::Tensor()};
    }
};

torch::autograd::variable_list TensorLinearFn::backward(torch::autograd::AutogradContext* ctx,
                                                        torch::autograd::variable_list grads) {
    const auto saved = ctx->get_saved_variables();
    const int64_t inds = ctx->saved_data["inds"].toInt();
    const at::Tensor &W = saved[0], &x = saved[1];
    const at::Tensor dy = grads[0].contiguous();
    at::Tensor dW, dx;
    // (needs_input_grad counts the tensor arguments only: W is 0, x is 1)
    if (ctx->needs_input_grad(0)) dW = WeightGradFn::apply(inds, dy, x, W.size(0), W.size(1));
    if (ctx->needs_input_grad(1)) dx = TensorLinearFn::apply(inds, W.t(), dy);
    return {at::Tensor(), dW, dx};
}

at::Tensor tensor_linear(int64_t inds, const at::Tensor& W, const at::Tensor& x) { return TensorLinearFn::apply(inds, W, x); }

// ------------------------------------------------------------------ TensorProds in one launch
// y = lin_o(prod(lin_l(x_l), lin_r(x_r))) (managan/tensor_products.py:109-121), for problems mg_tensor_prods_supported
// accepts; x: (..., dim, (3,)^inds), weights (out, in).  The module's forward is three such calls per a / v / d trio,
// node-sized: the host time of a call is what the caller sees.
bool tensor_prods_supported(int inds_l, int inds_r, int inds_o, int dim_l, int dim_r, int rank, int dim_o) {
    return mg_tensor_prods_supported(inds_l, inds_r, inds_o, dim_l, dim_r, rank, dim_o) != 0;
}

at::Tensor tensor_prods(int inds_l, int inds_r, int inds_o, const at::Tensor& W_l, const at::Tensor& W_r, const at::Tensor& W_o,
                        const at::Tensor& x_l_in, const at::Tensor& x_r_in) {
    const char* names[5] = {"W_l", "W_r", "W_o", "x_l", "x_r"};
    const at::Tensor* all[5] = {&W_l, &W_r, &W_o, &x_l_in, &x_r_in};
    for (int k = 0; k < 5; k++)
        TORCH_CHECK(all[k]->is_cuda() && all[k]->scalar_type() == at::kFloat, names[k], " must be a float32 CUDA tensor");
    TORCH_CHECK(W_l.dim() == 2 && W_r.dim() == 2 && W_o.dim() == 2, "weights must be matrices");
    TORCH_CHECK(inds_l >= 0 && inds_l <= 2 && inds_r >= 0 && inds_r <= 2 && inds_o >= 0 && inds_o <= 2, "ranks up to 2");
    const at::Tensor x_l = x_l_in.contiguous(), x_r = x_r_in.contiguous();
    const int64_t lead_l = x_l.dim() - inds_l - 1, lead_r = x_r.dim() - inds_r - 1;
    TORCH_CHECK(lead_l >= 0 && lead_l == lead_r && x_l.sizes().slice(0, lead_l) == x_r.sizes().slice(0, lead_r),
                "operands do not broadcast: ", x_l.sizes(), " vs ", x_r.sizes());
    const int64_t rank = W_l.size(0), dim_l = W_l.size(1), dim_r = W_r.size(1), dim_o = W_o.size(0);
    bool ok = x_l.size(lead_l) == dim_l && x_r.size(lead_r) == dim_r && W_r.size(0) == rank && W_o.size(1) == rank;
    for (int64_t k = lead_l + 1; k < x_l.dim(); k++) ok = ok && x_l.size(k) == 3;
    for (int64_t k = lead_r + 1; k < x_r.dim(); k++) ok = ok && x_r.size(k) == 3;
    TORCH_CHECK(ok, "shape mismatch between weights and operands");
    auto usable = [](const at::Tensor& W) {          // unit stride along a row, rows 16-byte aligned
        return (W.stride(1) == 1 && W.stride(0) % 4 == 0 && reinterpret_cast<uintptr_t>(W.data_ptr()) % 16 == 0) ? W
                                                                                                                 : W.contiguous();
    };
    const at::Tensor Wl = usable(W_l), Wr = usable(W_r), Wo = usable(W_o);
    int64_t rows = 1;
    std::vector<int64_t> y_shape;
    for (int64_t k = 0; k < lead_l; k++) { rows *= x_l.size(k); y_shape.push_back(x_l.size(k)); }
    y_shape.push_back(dim_o);
    for (int k = 0; k < inds_o; k++) y_shape.push_back(3);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(x_l.device());
    at::Tensor y = torch::empty(y_shape, x_l.options());
    check(mg_tensor_prods(inds_l, inds_r, inds_o, fp(Wl), Wl.stride(0), fp(Wr), Wr.stride(0), fp(Wo), Wo.stride(0), fp(x_l),
                          fp(x_r), rows, (int)dim_l, (int)dim_r, (int)rank, (int)dim_o, fp(y), stream_of(x_l)));
    return y;
}

// ------------------------------------------------------------------ codegen_tensops_cuda: Bee and Cow
std::vector<at::Tensor> bee_fwd(const at::Tensor& l_0, const at::Tensor& l_1, const at::Tensor& l_2, const at::Tensor& r_0,
                                const at::Tensor& r_1, const at::Tensor& r_2) {
    const auto [rows, chan] = rows_chan({&l_0, &l_1, &l_2}, {"l_0", "l_1", "l_2"});
    const auto rc = rows_chan({&r_0, &r_1, &r_2}, {"r_0", "r_1", "r_2"});
    TORCH_CHECK(rc.first == rows && rc.second == chan, "left and right operands must agree on batch and channel sizes");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(l_0.device());
    std::vector<at::Tensor> ys;
    std::array<float*, 13> ptrs{};
    for (int k = 0; k < 13; k++) {
        ys.push_back(torch::empty(shape_of(rows, chan, kBeeOrder[k][2] - '0'), l_0.options()));
        ptrs[k] = fp(ys.back());
    }
    check(mg_bee_fwd(fp(l_0), fp(l_1), fp(l_2), fp(r_0), fp(r_1), fp(r_2), rows, (int)chan, ptrs.data(), stream_of(l_0)));
    return ys;
}

std::vector<at::Tensor> bee_bwd(int side, const at::Tensor& o_0, const at::Tensor& o_1, const at::Tensor& o_2,
                                const std::vector<at::Tensor>& dys) {
    const auto [rows, chan] = rows_chan({&o_0, &o_1, &o_2}, {"x_0", "x_1", "x_2"});
    TORCH_CHECK(dys.size() == 13, "expected 13 output gradients");
    std::array<const float*, 13> ptrs{};
    for (int k = 0; k < 13; k++) {
        const std::string name = std::string("dy_") + kBeeOrder[k];
        check_input(dys[k], name.c_str());
        TORCH_CHECK(dys[k].sizes().vec() == shape_of(rows, chan, kBeeOrder[k][2] - '0'), name, " has wrong shape");
        ptrs[k] = fp(dys[k]);
    }
    c10::hip::HIPGuardMasqueradingAsCUDA guard(o_0.device());
    std::vector<at::Tensor> d;
    for (int k = 0; k < 3; k++) d.push_back(torch::empty(shape_of(rows, chan, k), o_0.options()));
    check(mg_bee_bwd(side, fp(o_0), fp(o_1), fp(o_2), ptrs.data(), rows, (int)chan, fp(d[0]), fp(d[1]), fp(d[2]),
                     stream_of(o_0)));
    return d;
}

std::pair<int64_t, int64_t> cow_inputs(const at::Tensor& l_0, const at::Tensor& l_1, const at::Tensor& r_0,
                                       const at::Tensor& r_1) {
    const auto lc = rows_chan({&l_0, &l_1}, {"l_0", "l_1"});
    const auto rc = rows_chan({&r_0, &r_1}, {"r_0", "r_1"});
    TORCH_CHECK(rc == lc, "left and right operands must agree on batch and channel sizes");
    return lc;
}

std::vector<at::Tensor> cow_o0_fwd(const at::Tensor& l_0, const at::Tensor& l_1, const at::Tensor& r_0, const at::Tensor& r_1) {
    const auto [rows, chan] = cow_inputs(l_0, l_1, r_0, r_1);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(l_0.device());
    at::Tensor y0 = torch::empty({rows, chan}, l_0.options()), y1 = torch::empty({rows, chan}, l_0.options());
    check(mg_cow_o0_fwd(fp(l_0), fp(l_1), fp(r_0), fp(r_1), rows, (int)chan, fp(y0), fp(y1), stream_of(l_0)));
    return {y0, y1};
}

std::vector<at::Tensor> cow_o1_fwd(const at::Tensor& l_0, const at::Tensor& l_1, const at::Tensor& r_0, const at::Tensor& r_1) {
    const auto [rows, chan] = cow_inputs(l_0, l_1, r_0, r_1);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(l_0.device());
    std::vector<at::Tensor> ys;
    for (int k = 0; k < 3; k++) ys.push_back(torch::empty({rows, chan, 3}, l_0.options()));
    check(mg_cow_o1_fwd(fp(l_0), fp(l_1), fp(r_0), fp(r_1), rows, (int)chan, fp(ys[0]), fp(ys[1]), fp(ys[2]), stream_of(l_0)));
    return ys;
}

std::vector<at::Tensor> cow_bwd(int which, int side, const at::Tensor& o_0, const at::Tensor& o_1,
                                const std::vector<at::Tensor>& dys) {
    const auto [rows, chan] = rows_chan({&o_0, &o_1}, {"x_0", "x_1"});
    const size_t want = which == 0 ? 2 : 3;
    TORCH_CHECK(dys.size() == want, "wrong number of output gradients");
    for (size_t k = 0; k < want; k++) {
        const std::string name = "dy[" + std::to_string(k) + "]";
        check_input(dys[k], name.c_str());
        TORCH_CHECK(dys[k].sizes().vec() == shape_of(rows, chan, which), name, " has wrong shape");
    }
    c10::hip::HIPGuardMasqueradingAsCUDA guard(o_0.device());
    at::Tensor d0 = torch::empty({rows, chan}, o_0.options()), d1 = torch::empty({rows, chan, 3}, o_0.options());
    if (which == 0)
        check(mg_cow_o0_bwd(side, fp(o_0), fp(o_1), fp(dys[0]), fp(dys[1]), rows, (int)chan, fp(d0), fp(d1), stream_of(o_0)));
    else
        check(mg_cow_o1_bwd(side, fp(o_0), fp(o_1), fp(dys[0]), fp(dys[1]), fp(dys[2]), rows, (int)chan, fp(d0), fp(d1),
                            stream_of(o_0)));
    return {d0, d1};
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "torch C++ binding of libmanagan_hip.so with the signatures of the reference's compiled extensions";
    // neighbour_grid_cuda (neighbour_grid.cpp:198-203)
    m.def("get_neighbours", &get_neighbours, "Define neighbours based on cutoff radius using a grid method.");
    m.def("edges_read", &edges_read, "Read data from nodes to edges.");
    m.def("edges_reduce", &edges_reduce, "Reduce data from edges to nodes.");
    m.def("get_edges", &get_edges, "Like get_neighbours, except it returns lists of edge tensors.");
    // tensor_ops_cuda (tensor_ops.cpp:180-182)
    m.def("tensor_linear", &tensor_linear, "tensor_linear(inds, W, x)");
    // TensorProds.forward (managan/tensor_products.py:109-121) as one launch
    m.def("tensor_prods_supported", &tensor_prods_supported);
    m.def("tensor_prods", &tensor_prods, "lin_o(prod(lin_l(x_l), lin_r(x_r)))");
    // codegen_tensops_cuda (codegen_tensops.cpp:2001-2010): the gradients arrive as positional arguments
    m.def("bee_fwd_cuda", &bee_fwd);
    m.def("bee_bwl_cuda", [](const at::Tensor& r_0, const at::Tensor& r_1, const at::Tensor& r_2, const py::args& dys) {
        return bee_bwd(0, r_0, r_1, r_2, dys.cast<std::vector<at::Tensor>>());
    });
    m.def("bee_bwr_cuda", [](const at::Tensor& l_0, const at::Tensor& l_1, const at::Tensor& l_2, const py::args& dys) {
        return bee_bwd(1, l_0, l_1, l_2, dys.cast<std::vector<at::Tensor>>());
    });
    m.def("cow_o0_fwd_cuda", &cow_o0_fwd);
    m.def("cow_o1_fwd_cuda", &cow_o1_fwd);
    m.def("cow_o0_bwl_cuda", [](const at::Tensor& r_0, const at::Tensor& r_1, const py::args& dys) {
        return cow_bwd(0, 0, r_0, r_1, dys.cast<std::vector<at::Tensor>>());
    });
    m.def("cow_o0_bwr_cuda", [](const at::Tensor& l_0, const at::Tensor& l_1, const py::args& dys) {
        return cow_bwd(0, 1, l_0, l_1, dys.cast<std::vector<at::Tensor>>());
    });
    m.def("cow_o1_bwl_cuda", [](const at::Tensor& r_0, const at::Tensor& r_1, const py::args& dys) {
        return cow_bwd(1, 0, r_0, r_1, dys.cast<std::vector<at::Tensor>>());
    });
    m.def("cow_o1_bwr_cuda", [](const at::Tensor& l_0, const at::Tensor& l_1, const py::args& dys) {
        return cow_bwd(1, 1, l_0, l_1, dys.cast<std::vector<at::Tensor>>());
    });
}
