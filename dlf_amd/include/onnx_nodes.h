// Host veneer: the ONNX node operators that land on the axis primitives, as dlf's
// interpreter builds them for a GPU context (dlf/include/predict.h: ReductionOp :1078-1097
// and its ten node kinds :1099-1137, ArgMaxOp / ArgMinOp :1139-1177, CumSumOp :1179-1201,
// TopKOp :1486-1510, NonZeroOp :2031-2044, and the Softmax / LogSoftmax / Hardmax nodes
// over dnn::softmax / logsoftmax / hardmax).
//
// The reference's operators are bound to a model::Node (attributes) and to datum slots
// (tensors) by an OperatorFactory and then run by evaluate().  The same three pieces are here
// without the model IR: a Node carries the operator name, its attributes and pointers to its
// input and output device tensors; make_operator() does what the factory's visit() overloads
// do (reads the attributes with the reference's defaults, once); Operator::evaluate() issues
// the front-end call.  Tensor-valued inputs that the reference reads on the host at
// evaluation time (CumSum's axis, TopK's K) are host tensors here.
#pragma once

#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "dev_tensor.h"

namespace dlf { namespace predict {

// Attribute access with defaults, as model::Node::get_i / get_is.
class Attributes {
    std::map<std::string, int64_t> ints_;
    std::map<std::string, std::vector<int64_t>> int_lists_;
public:
    Attributes& set_i(const std::string& name, int64_t v) { ints_[name] = v; return *this; }
    Attributes& set_is(const std::string& name, std::vector<int64_t> v) { int_lists_[name] = std::move(v); return *this; }
    int64_t get_i(const std::string& name, int64_t fallback) const {
        auto it = ints_.find(name);
        return it == ints_.end() ? fallback : it->second;
    }
    std::vector<int64_t> get_is(const std::string& name, std::vector<int64_t> fallback) const {
        auto it = int_lists_.find(name);
        return it == int_lists_.end() ? fallback : it->second;
    }
};

// One node of a graph whose tensors have element type T: inputs / outputs of that type,
// 32-bit integer outputs (ArgMax, ArgMin, TopK indices, NonZero) and host-read inputs.
template <typename T>
struct Node {
    std::string op_type;
    Attributes attrs;
    std::vector<const DevTensor<T>*> inputs;
    std::vector<const Tensor<int64_t>*> host_inputs;     // CumSum: axis (rank 0); TopK: K (one element)
    std::vector<DevTensor<T>*> outputs;
    std::vector<DevTensor<int32_t>*> index_outputs;
};

struct Operator {
    virtual ~Operator() = default;
    virtual void evaluate() = 0;
};

class unsupported_operator : public std::invalid_argument {
public:
    using std::invalid_argument::invalid_argument;
};

namespace detail {

inline const char* reducer_of(const std::string& op_type) {      // predict.h:1099-1137
    static const std::map<std::string, const char*> table = {
        {"ReduceMax", "reduce_max"}, {"ReduceMin", "reduce_min"}, {"ReduceSum", "reduce_sum"},
        {"ReduceSumSquare", "reduce_sum_square"}, {"ReduceMean", "reduce_mean"}, {"ReduceProd", "reduce_prod"},
        {"ReduceLogSum", "reduce_log_sum"}, {"ReduceLogSumExp", "reduce_log_sum_exp"},
        {"ReduceL1", "reduce_asum"}, {"ReduceL2", "reduce_nrm2"}};
    auto it = table.find(op_type);
    return it == table.end() ? nullptr : it->second;
}

template <typename P>
P* need(const std::vector<P*>& v, size_t i, const char* what) {
    if (i >= v.size() || !v[i]) throw std::invalid_argument(std::string("node is missing ") + what);
    return v[i];
}

template <typename T>
struct ReductionOp : Operator {                      // predict.h:1078-1097
    const DevTensor<T>* X;
    DevTensor<T>* Y;
    std::string reducer;
    std::vector<int> axes;
    bool keepdims;
    ReductionOp(const Node<T>& n, const char* name)
        : X(need(n.inputs, 0, "its input")), Y(need(n.outputs, 0, "its output")), reducer(name) {
        for (int64_t a : n.attrs.get_is("axes", {})) axes.push_back(static_cast<int>(a));     // default: every axis
        keepdims = n.attrs.get_i("keepdims", 1) != 0;
    }
    void evaluate() override { dlf::reduce(reducer, *X, *Y, axes, keepdims); }
};

template <typename T>
struct ArgReduceOp : Operator {                      // predict.h:1139-1177
    const DevTensor<T>* X;
    DevTensor<int32_t>* Y;
    const char* name;
    int axis;
    bool keepdims;
    ArgReduceOp(const Node<T>& n, const char* fn)
        : X(need(n.inputs, 0, "its input")), Y(need(n.index_outputs, 0, "its index output")), name(fn),
          axis(static_cast<int>(n.attrs.get_i("axis", 0))), keepdims(n.attrs.get_i("keepdims", 1) != 0) {}
    void evaluate() override { dlf::detail::arg_reduce(*X, *Y, axis, keepdims, name); }
};

template <typename T>
struct CumSumOp : Operator {                         // predict.h:1179-1201
    const DevTensor<T>* X;
    DevTensor<T>* Y;
    const Tensor<int64_t>* axis;
    bool exclusive, reverse;
    explicit CumSumOp(const Node<T>& n)
        : X(need(n.inputs, 0, "its input")), Y(need(n.outputs, 0, "its output")), axis(need(n.host_inputs, 0, "its axis input")),
          exclusive(n.attrs.get_i("exclusive", 0) != 0), reverse(n.attrs.get_i("reverse", 0) != 0) {}
    void evaluate() override {
        if (axis->size() != 1) throw shape_error("CumSum: axis must hold one element");
        dlf::cumsum(*X, *Y, static_cast<int>(axis->values()[0]), exclusive, reverse);      // Y may be X (in place)
    }
};

template <typename T>
struct TopKOp : Operator {                           // predict.h:1486-1510
    const DevTensor<T>* X;
    DevTensor<T>* Y;
    DevTensor<int32_t>* I;
    const Tensor<int64_t>* K;
    int axis;
    bool largest;
    explicit TopKOp(const Node<T>& n)
        : X(need(n.inputs, 0, "X")), Y(need(n.outputs, 0, "Y")), I(need(n.index_outputs, 0, "its index output")),
          K(need(n.host_inputs, 0, "K")), axis(static_cast<int>(n.attrs.get_i("axis", -1))),
          largest(n.attrs.get_i("largest", 1) != 0) {}
    // `sorted` is read by the reference and ignored by its device path (reorder_detail.h:1066);
    // the output here is always sorted.
    void evaluate() override {
        if (K->size() != 1 || K->values()[0] < 0) throw shape_error("TopK: K must be one non-negative element");
        dlf::top_k(*X, *Y, *I, static_cast<size_t>(K->values()[0]), axis, largest);
    }
};

template <typename T>
struct NonZeroOp : Operator {                        // predict.h:2031-2044: [rank, n]
    const DevTensor<T>* X;
    DevTensor<int32_t>* Y;
    explicit NonZeroOp(const Node<T>& n) : X(need(n.inputs, 0, "its input")), Y(need(n.index_outputs, 0, "its index output")) {}
    void evaluate() override { dlf::nonzero(*X, *Y, true); }
};

template <typename T>
struct RowNormalizeOp : Operator {                   // Softmax / LogSoftmax / Hardmax nodes, axis default 1
    const DevTensor<T>* X;
    DevTensor<T>* Y;
    int kind, axis;
    RowNormalizeOp(const Node<T>& n, int k)
        : X(need(n.inputs, 0, "its input")), Y(need(n.outputs, 0, "its output")), kind(k),
          axis(static_cast<int>(n.attrs.get_i("axis", 1))) {}
    void evaluate() override {
        if (kind == 0) dlf::dnn::softmax(*X, *Y, axis);
        else if (kind == 1) dlf::dnn::logsoftmax(*X, *Y, axis);
        else dlf::dnn::hardmax(*X, *Y, axis);
    }
};

}  // namespace detail

// What OperatorFactory::visit does for these node kinds: reads the attributes and binds the
// tensors.  Throws unsupported_operator for a node that is not one of the axis primitives.
template <typename T>
std::unique_ptr<Operator> make_operator(const Node<T>& n) {
    if (const char* reducer = detail::reducer_of(n.op_type)) return std::make_unique<detail::ReductionOp<T>>(n, reducer);
    if (n.op_type == "ArgMax") return std::make_unique<detail::ArgReduceOp<T>>(n, "argmax");
    if (n.op_type == "ArgMin") return std::make_unique<detail::ArgReduceOp<T>>(n, "argmin");
    if (n.op_type == "CumSum") return std::make_unique<detail::CumSumOp<T>>(n);
    if (n.op_type == "TopK") return std::make_unique<detail::TopKOp<T>>(n);
    if (n.op_type == "NonZero") return std::make_unique<detail::NonZeroOp<T>>(n);
    if (n.op_type == "Softmax") return std::make_unique<detail::RowNormalizeOp<T>>(n, 0);
    if (n.op_type == "LogSoftmax") return std::make_unique<detail::RowNormalizeOp<T>>(n, 1);
    if (n.op_type == "Hardmax") return std::make_unique<detail::RowNormalizeOp<T>>(n, 2);
    throw unsupported_operator("operator " + n.op_type + " is not one of the axis primitives");
}

// Builds and runs one node (the interpreter's loop body for a single operator).
template <typename T>
void evaluate(const Node<T>& n) { make_operator(n)->evaluate(); }

}}  // namespace dlf::predict
