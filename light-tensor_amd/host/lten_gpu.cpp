// See lten_gpu.h.  Every GPU branch is a call through the C ABI of liblten_hip (include/lten_hip.h);
// the l-ten source line each one stands in for is cited beside it.
#include "lten_gpu.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>

#include "../../include/lten_hip.h"

namespace lten {

// ------------------------------------------------------------------------------ errors

ExceptionInfo::ExceptionInfo(const char* msg, const char* file, const char* func, int line)
{
	char buf[1024];
	snprintf(buf, sizeof(buf), "%s [%s %s:%d]", msg, func, file, line);
	text_ = buf;
}

void ltenFail(const char* msg, const char* file, const char* func, int line)
{
	// l-ten prints, then throws (l-ten/error.h:91-93, l-ten/utils.cpp:303-321)
	fprintf(stderr, "[Error] File: %s Function: %s Line:%d Msg: %s\n", file, func, line, msg);
	throw ExceptionInfo(msg, file, func, line);
}

// a non-zero status of the C ABI becomes an l-ten error, message included
#define LTEN_HIP_CALL(expr)                                  \
	do {                                                 \
		if ((expr) != 0) LTEN_ERR(lten_hip_last_error()); \
	} while (0)

// ------------------------------------------------------------------------------ TensorImpl

static size_t elem_size(dtype t) { return t == UINT8 ? 1 : 4; }

struct TensorImpl {
	uint64_t dims[MAX_DIMS] = { 0 };
	int ndims = 0;
	uint64_t numels = 0;
	dtype data_type = FLOAT32;
	device dev = CPU;
	int dev_index = 0;
	void* data = nullptr;
	bool own_data = false;
	void* grad = nullptr;
	bool autograd = false;
	std::vector<std::shared_ptr<TensorImpl>> children;
	grad_fn_t grad_fn;

	size_t nbytes() const { return numels * elem_size(data_type); }

	static void* alloc(device d, size_t bytes, bool zero)
	{
		if (d == CPU) return zero ? calloc(bytes ? bytes : 1, 1) : malloc(bytes ? bytes : 1);
		void* p = nullptr;
		LTEN_HIP_CALL(lten_hip_alloc(&p, bytes, zero ? 1 : 0));  // l-ten/utils.cu:30-58 AllocateMemoryOnGPU
		return p;
	}
	static void release(device d, void* p)
	{
		if (!p) return;
		if (d == CPU) free(p);
		else lten_hip_free(p);  // l-ten/utils.cu:60-71
	}
	void ensure_grad()
	{
		if (!grad) grad = alloc(dev, nbytes(), true);
	}
	~TensorImpl()
	{
		if (own_data) release(dev, data);
		release(dev, grad);
	}
};

static std::shared_ptr<TensorImpl> make_impl(const uint64_t* dims, int ndims, void* data, bool own, const TensorOps* ops)
{
	if (ndims < 1 || ndims > MAX_DIMS) LTEN_ERR("Invalid number of dimensions");
	auto t = std::make_shared<TensorImpl>();
	TensorOps def;
	if (!ops) ops = &def;
	t->ndims = ndims;
	t->numels = 1;
	for (int i = 0; i < ndims; i++) {
		t->dims[i] = dims[i];
		t->numels *= dims[i];
	}
	t->data_type = ops->data_type;
	t->dev = ops->device_type;
	t->dev_index = ops->device_index;
	if (t->dev == GPU) LTEN_HIP_CALL(lten_hip_init(t->dev_index));
	if (data) {
		t->data = data;
		t->own_data = own;
	} else {
		t->data = TensorImpl::alloc(t->dev, t->nbytes(), false);
		t->own_data = true;
	}
	if (ops->alloc_gradient_buffer) t->ensure_grad();
	return t;
}

// ------------------------------------------------------------------------------ Tensor

void* Tensor::get_data_ptr() { return impl_->data; }
void* Tensor::get_grad_ptr() { return impl_->grad; }
uint64_t Tensor::get_numels() const { return impl_->numels; }
const uint64_t* Tensor::get_sizes() const { return impl_->dims; }
int Tensor::get_ndims() const { return impl_->ndims; }
dtype Tensor::get_data_type() const { return impl_->data_type; }
device Tensor::get_device() const { return impl_->dev; }
int Tensor::get_device_index() const { return impl_->dev_index; }
void Tensor::set_autograd(bool setting) { impl_->autograd = setting; }

void Tensor::clear_gradients()
{
	if (!impl_->grad) return;
	if (impl_->dev == CPU) memset(impl_->grad, 0, impl_->nbytes());
	else LTEN_HIP_CALL(lten_hip_zero(impl_->grad, impl_->nbytes()));  // l-ten/utils.cu:49-52 ZeroMemoryOnGPU
}

Tensor TensorFromBuffer(const uint64_t* dims_ptr, int ndims, void* data_ptr, bool own_memory, TensorOps* options_ptr)
{
	return Tensor(make_impl(dims_ptr, ndims, data_ptr, own_memory, options_ptr));
}
Tensor TensorFromBuffer(const std::initializer_list<uint64_t>& dims, void* data_ptr, bool own_memory, TensorOps* options_ptr)
{
	return TensorFromBuffer(dims.begin(), (int)dims.size(), data_ptr, own_memory, options_ptr);
}
Tensor AllocateTensor(const uint64_t* dims_ptr, int ndims, TensorOps* options_ptr)
{
	return TensorFromBuffer(dims_ptr, ndims, nullptr, true, options_ptr);
}
Tensor AllocateTensor(const std::initializer_list<uint64_t>& dims, TensorOps* options_ptr)
{
	return TensorFromBuffer(dims.begin(), (int)dims.size(), nullptr, true, options_ptr);
}

static void copy_between(device dst_dev, void* dst, device src_dev, const void* src, size_t bytes)
{
	if (bytes == 0) return;
	if (dst_dev == CPU && src_dev == CPU) memcpy(dst, src, bytes);
	else if (dst_dev == GPU && src_dev == CPU) LTEN_HIP_CALL(lten_hip_copy_to_gpu(dst, src, bytes));        // l-ten/utils.cu:73-80
	else if (dst_dev == CPU && src_dev == GPU) LTEN_HIP_CALL(lten_hip_copy_from_gpu(dst, src, bytes));      // l-ten/utils.cu:82-94
	else LTEN_HIP_CALL(lten_hip_copy_gpu_to_gpu(dst, src, bytes));                                         // l-ten/utils.cu:96-108
}

Tensor Tensor::to(device target_device, int target_device_index)
{
	// l-ten/tensorimpl.cpp:311-412: data and, when present, the gradient buffer move together
	TensorOps ops;
	ops.data_type = impl_->data_type;
	ops.device_type = target_device;
	ops.device_index = target_device_index;
	Tensor out = AllocateTensor(impl_->dims, impl_->ndims, &ops);
	copy_between(target_device, out.impl_->data, impl_->dev, impl_->data, impl_->nbytes());
	if (impl_->grad) {
		out.impl_->ensure_grad();
		copy_between(target_device, out.impl_->grad, impl_->dev, impl_->grad, impl_->nbytes());
	}
	out.impl_->autograd = impl_->autograd;
	return out;
}

// Where a child's gradient goes: straight into its own (zero-initialised, accumulating) gradient buffer when
// it is a leaf, into a fresh zeroed buffer when it is an intermediate result that has to be propagated further.
struct Bottom {
	std::shared_ptr<TensorImpl> child;
	float* ptr = nullptr;
	bool temporary = false;
	explicit Bottom(const std::shared_ptr<TensorImpl>& c) : child(c)
	{
		if (c->grad_fn) {
			ptr = static_cast<float*>(TensorImpl::alloc(c->dev, c->nbytes(), true));
			temporary = true;
		} else {
			c->ensure_grad();
			ptr = static_cast<float*>(c->grad);
		}
	}
	void propagate()
	{
		if (temporary) {
			child->grad_fn(*child, ptr);
			if (child->dev == GPU) LTEN_HIP_CALL(lten_hip_sync());
			TensorImpl::release(child->dev, ptr);
			temporary = false;
		}
	}
};
static bool wants_gradient(const std::shared_ptr<TensorImpl>& c) { return c->autograd || (bool)c->grad_fn; }

void Tensor::backward(const Tensor* top_gradient)
{
	if (impl_->data_type != FLOAT32) LTEN_ERR("backward is only supported for FLOAT32 tensors");
	if (!impl_->grad_fn) return;
	if (top_gradient) {
		if (top_gradient->get_numels() != impl_->numels || top_gradient->get_device() != impl_->dev)
			LTEN_ERR("top gradient must have the shape and device of the tensor");
		impl_->grad_fn(*impl_, static_cast<const float*>(top_gradient->impl_->data));
		return;
	}
	if (impl_->numels != 1) LTEN_ERR("backward without a top gradient needs a one-element tensor");
	float one = 1.0f;
	TensorOps ops;
	Tensor seed = TensorFromBuffer({ 1 }, &one, false, &ops).to(impl_->dev, impl_->dev_index);
	impl_->grad_fn(*impl_, static_cast<const float*>(seed.impl_->data));
}

// ------------------------------------------------------------------------------ matmul

static void leading_offsets(const TensorImpl& a, const TensorImpl& b, const uint64_t* cdims, int ndims, std::vector<uint64_t>& oa,
                            std::vector<uint64_t>& ob)
{
	// l-ten/md_array.h:1252-1282: broadcast = coordinate clamped to dim - 1
	uint64_t count = 1;
	for (int i = 0; i < ndims - 2; i++) count *= cdims[i];
	oa.resize(count);
	ob.resize(count);
	const uint64_t ma = a.dims[ndims - 2] * a.dims[ndims - 1], mb = b.dims[ndims - 2] * b.dims[ndims - 1];
	for (uint64_t idx = 0; idx < count; idx++) {
		uint64_t rem = idx, offa = 0, offb = 0, sa = 1, sb = 1;
		for (int i = ndims - 3; i >= 0; i--) {
			const uint64_t c = rem % cdims[i];
			rem /= cdims[i];
			offa += (c < a.dims[i] ? c : a.dims[i] - 1) * sa;
			offb += (c < b.dims[i] ? c : b.dims[i] - 1) * sb;
			sa *= a.dims[i];
			sb *= b.dims[i];
		}
		oa[idx] = offa * ma;
		ob[idx] = offb * mb;
	}
}

// True when the operand offsets of consecutive leading indices advance by constant strides (stride 0 = one operand
// broadcast over every leading dim), so that one strided-batched launch covers the loop.
static bool uniform_strides(const std::vector<uint64_t>& oa, const std::vector<uint64_t>& ob, int64_t& sa, int64_t& sb)
{
	sa = oa.size() > 1 ? (int64_t)oa[1] : 0;
	sb = ob.size() > 1 ? (int64_t)ob[1] : 0;
	for (size_t i = 0; i < oa.size(); i++)
		if (oa[i] != (uint64_t)sa * i || ob[i] != (uint64_t)sb * i) return false;
	return true;
}

Tensor Tensor::matmul(const Tensor& other)
{
	TensorImpl& a = *impl_;
	TensorImpl& b = *other.impl_;
	if (a.data_type != b.data_type) LTEN_ERR("Tensor data types must match");                       // l-ten/tensor.h:87-90
	if (a.data_type != FLOAT32) LTEN_ERR("Not yet implemented");                                    // l-ten/math_fns.cpp:1295-1305
	if (a.ndims != b.ndims) LTEN_ERR("MultiDimArrays must have the same number of dimensions");    // l-ten/md_array.h:971-974
	if (a.dev != b.dev || a.dev_index != b.dev_index) LTEN_ERR("Tensors must be on the same device");
	if (a.ndims < 2) LTEN_ERR("matmul requires at least 2 dimensions");
	const int nd = a.ndims;
	if (a.dims[nd - 1] != b.dims[nd - 2]) LTEN_ERR("MultiDimArrays must have compatiple dimensions");  // l-ten/md_array.h:985-988
	uint64_t cdims[MAX_DIMS];
	for (int i = 0; i < nd - 2; i++) {
		if (a.dims[i] != b.dims[i] && a.dims[i] != 1 && b.dims[i] != 1) LTEN_ERR("MultiDimArrays must have compatiple dimensions");
		cdims[i] = a.dims[i] > b.dims[i] ? a.dims[i] : b.dims[i];
	}
	const uint64_t M = a.dims[nd - 2], K = a.dims[nd - 1], N = b.dims[nd - 1];
	cdims[nd - 2] = M;
	cdims[nd - 1] = N;
	if (a.dev != GPU) LTEN_ERR("this build implements matmul for the GPU device type only (l-ten's own CPU path covers lten::CPU)");

	TensorOps ops;
	ops.device_type = GPU;
	ops.device_index = a.dev_index;
	Tensor result = AllocateTensor(cdims, nd, &ops);
	std::vector<uint64_t> oa, ob;
	leading_offsets(a, b, cdims, nd, oa, ob);
	const float* ad = static_cast<const float*>(a.data);
	const float* bd = static_cast<const float*>(b.data);
	float* cd = static_cast<float*>(result.impl_->data);
	// l-ten/md_array_cuda.h:507-515 runs one NN GEMM per leading index.  When the operand offsets advance by a constant
	// stride (no broadcast, or one operand broadcast over all leading dims: stride 0) the whole loop is one launch.
	int64_t sa = 0, sb = 0;
	const bool uniform = uniform_strides(oa, ob, sa, sb);
	if (uniform)
		LTEN_HIP_CALL(lten_hip_sgemm_strided_batched(0, 0, M, N, K, 1.0f, ad, K, sa, bd, N, sb, 0.0f, cd, N, (int64_t)(M * N), oa.size()));
	else
		for (size_t i = 0; i < oa.size(); i++)
			LTEN_HIP_CALL(lten_hip_sgemm(0, 0, M, N, K, 1.0f, ad + oa[i], K, bd + ob[i], N, 0.0f, cd + i * M * N, N));

	auto ai = impl_, bi = other.impl_;
	result.impl_->children = { ai, bi };
	result.impl_->autograd = true;
	result.impl_->grad_fn = [ai, bi, oa, ob, M, N, K, uniform, sa, sb](TensorImpl& self, const float* top) {
		(void)self;
		// l-ten/backprop.cpp:533-585: per leading index dA += dC B^T (NT), dB += A^T dC (TN), beta = 1 into
		// zeroed gradients, so a broadcast operand collects the sum over the indices that share it
		const float* ad = static_cast<const float*>(ai->data);
		const float* bd = static_cast<const float*>(bi->data);
		if (wants_gradient(ai)) {
			Bottom g(ai);
			if (uniform)
				LTEN_HIP_CALL(lten_hip_sgemm_strided_batched(0, 1, M, K, N, 1.0f, top, N, (int64_t)(M * N), bd, N, sb, 1.0f, g.ptr, K, sa, oa.size()));
			else
				for (size_t i = 0; i < oa.size(); i++)
					LTEN_HIP_CALL(lten_hip_sgemm(0, 1, M, K, N, 1.0f, top + i * M * N, N, bd + ob[i], N, 1.0f, g.ptr + oa[i], K));
			g.propagate();
		}
		if (wants_gradient(bi)) {
			Bottom g(bi);
			if (uniform)
				LTEN_HIP_CALL(lten_hip_sgemm_strided_batched(1, 0, K, N, M, 1.0f, ad, K, sa, top, N, (int64_t)(M * N), 1.0f, g.ptr, N, sb, oa.size()));
			else
				for (size_t i = 0; i < oa.size(); i++)
					LTEN_HIP_CALL(lten_hip_sgemm(1, 0, K, N, M, 1.0f, ad + oa[i], K, top + i * M * N, N, 1.0f, g.ptr + ob[i], N));
			g.propagate();
		}
	};
	return result;
}

// ------------------------------------------------------------------------------ FullyConnected

static void check_layer_input(const Tensor& input, Tensor& weight, const char* what)
{
	// l-ten/fully_connected.cpp:73-78
	if (input.get_device() != weight.get_device() || input.get_device_index() != weight.get_device_index() ||
	    input.get_data_type() != weight.get_data_type())
		LTEN_ERR("Input tensor device type or data type are not the same as this layer's parameters");
	(void)what;
}

bool FullyConnected::init()
{
	// l-ten/fully_connected.cpp:9-55: weight {1,1,out,in}, bias {out}, U(-sqrt(1/in), sqrt(1/in)) from std::random_device
	TensorOps options;
	weight_ = AllocateTensor({ 1, 1, output_features_, input_features_ }, &options);
	weight_.set_autograd(true);
	std::random_device generator;
	std::uniform_real_distribution<float> distribution(-sqrtf(1.0f / input_features_), sqrtf(1.0f / input_features_));
	float* w = static_cast<float*>(weight_.get_data_ptr());
	for (uint64_t i = 0; i < weight_.get_numels(); i++) w[i] = distribution(generator);
	if (use_bias_) {
		options.alloc_gradient_buffer = true;
		bias_ = AllocateTensor({ output_features_ }, &options);
		bias_.set_autograd(true);
		float* b = static_cast<float*>(bias_.get_data_ptr());
		for (uint64_t i = 0; i < bias_.get_numels(); i++) b[i] = distribution(generator);
	}
	return true;
}

void FullyConnected::to(device target_device, int target_device_index)
{
	// l-ten/fully_connected.cpp:220-289; the bias_multiplier ones vector of l-ten is not needed: the bias is
	// added in the GEMM epilogue and its gradient is a column sum that needs no operand of ones
	if (weight_.defined()) weight_ = weight_.to(target_device, target_device_index);
	if (use_bias_ && bias_.defined()) bias_ = bias_.to(target_device, target_device_index);
}

void FullyConnected::clear_gradients()
{
	if (weight_.defined()) weight_.clear_gradients();
	if (use_bias_ && bias_.defined()) bias_.clear_gradients();
}

std::vector<Tensor*> FullyConnected::get_all_weights()
{
	std::vector<Tensor*> w{ &weight_ };
	if (use_bias_) w.push_back(&bias_);
	return w;
}

Tensor FullyConnected::forward(Tensor& input)
{
	const int ndims = input.get_ndims();
	if (ndims < 3) LTEN_ERR("FullyConnected requires tensors with at least 3 dimensions");  // l-ten/fully_connected.cpp:68-71
	check_layer_input(input, weight_, "FullyConnected");
	uint64_t dims[MAX_DIMS];
	memcpy(dims, input.get_sizes(), sizeof(uint64_t) * ndims);
	if (dims[ndims - 1] != input_features_) LTEN_ERR("Last dimension must be equal to the number of input features");  // :82-85
	dims[ndims - 1] = output_features_;
	if (input.get_device() != GPU)
		LTEN_ERR("this build implements FullyConnected for the GPU device type only (l-ten's own CPU path covers lten::CPU)");

	TensorOps options;
	options.data_type = input.get_data_type();
	options.device_index = input.get_device_index();
	options.device_type = GPU;
	Tensor result = AllocateTensor(dims, ndims, &options);
	uint64_t M = 1;  // l-ten/fully_connected.cpp:100-104: all leading dims folded into one GEMM
	for (int i = 0; i < ndims - 1; i++) M *= dims[i];
	// l-ten/fully_connected.cpp:150 (NT GEMM) + :165 (bias as a rank-1 GEMM), one launch here
	LTEN_HIP_CALL(lten_hip_fc_forward_f32(M, input_features_, output_features_, static_cast<const float*>(input.get_data_ptr()),
	                                      static_cast<const float*>(weight_.get_data_ptr()),
	                                      use_bias_ ? static_cast<const float*>(bias_.get_data_ptr()) : nullptr,
	                                      static_cast<float*>(result.get_data_ptr())));
	if (is_training_) {
		auto in = input.get_smart_ptr(), wt = weight_.get_smart_ptr();
		std::shared_ptr<TensorImpl> bs = use_bias_ ? bias_.get_smart_ptr() : nullptr;
		const uint64_t fin = input_features_, fout = output_features_;
		result.get_smart_ptr()->children = { in, wt };  // l-ten/fully_connected.cpp:181-184
		result.get_smart_ptr()->autograd = true;
		result.get_smart_ptr()->grad_fn = [in, wt, bs, M, fin, fout](TensorImpl&, const float* top) {
			const float* x = static_cast<const float*>(in->data);
			const float* w = static_cast<const float*>(wt->data);
			if (wants_gradient(in)) {  // l-ten/backprop.cpp:2228  dX = dY W (NN)
				Bottom g(in);
				LTEN_HIP_CALL(lten_hip_sgemm(0, 0, M, fin, fout, 1.0f, top, fout, w, fin, 1.0f, g.ptr, fin));
				g.propagate();
			}
			if (wants_gradient(wt)) {  // l-ten/backprop.cpp:2252  dW = dY^T X (TN)
				Bottom g(wt);
				LTEN_HIP_CALL(lten_hip_sgemm(1, 0, fout, fin, M, 1.0f, top, fout, x, fin, 1.0f, g.ptr, fin));
			}
			if (bs) {  // l-ten/backprop.cpp:2267  db += ones dY, straight into the bias gradient buffer
				bs->ensure_grad();
				LTEN_HIP_CALL(lten_hip_fc_backward_f32(M, fin, fout, x, w, top, nullptr, nullptr, static_cast<float*>(bs->grad)));
			}
		};
	}
	return result;
}

// ------------------------------------------------------------------------------ relu, log_softmax, nll_loss

static void require_gpu_f32(const Tensor& t, const char* what)
{
	if (t.get_data_type() != FLOAT32) LTEN_ERR("Not yet implemented");
	if (t.get_device() != GPU) {
		static std::string msg;
		msg = std::string("this build implements ") + what + " for the GPU device type only (l-ten's own CPU path covers lten::CPU)";
		LTEN_ERR(msg.c_str());
	}
}

Tensor Tensor::reshape(const std::initializer_list<uint64_t>& dims)
{
	uint64_t count = 1;
	for (uint64_t d : dims) count *= d;
	if (count != impl_->numels) LTEN_ERR("reshape: the number of elements must stay the same");
	TensorOps options;
	options.data_type = impl_->data_type;
	options.device_type = impl_->dev;
	options.device_index = impl_->dev_index;
	Tensor result = TensorFromBuffer(dims, impl_->data, false, &options);
	auto in = impl_;
	result.get_smart_ptr()->children = { in };  // keeps the shared buffer alive (l-ten/tensorimpl.cpp:2044)
	if (wants_gradient(in)) {
		if (impl_->data_type != FLOAT32) LTEN_ERR("reshape: gradients are implemented for FLOAT32 tensors only");
		const uint64_t n = impl_->numels;
		result.get_smart_ptr()->autograd = true;
		result.get_smart_ptr()->grad_fn = [in, n](TensorImpl&, const float* top) {  // l-ten/backprop.cpp:2475-2505: a copy of the top gradient
			if (in->grad_fn) {
				in->grad_fn(*in, top);  // same values, same order: handed on as it is
			} else {
				in->ensure_grad();
				if (in->dev == GPU) LTEN_HIP_CALL(lten_hip_axpy_f32(n, 1.0f, top, static_cast<float*>(in->grad)));
				else for (uint64_t i = 0; i < n; i++) static_cast<float*>(in->grad)[i] += top[i];
			}
		};
	}
	return result;
}

Tensor relu(Tensor& input)
{
	require_gpu_f32(input, "relu");
	TensorOps options;
	options.device_index = input.get_device_index();
	options.device_type = GPU;
	Tensor result = AllocateTensor(input.get_sizes(), input.get_ndims(), &options);
	const uint64_t n = input.get_numels();
	LTEN_HIP_CALL(lten_hip_relu_f32(static_cast<float*>(result.get_data_ptr()), static_cast<const float*>(input.get_data_ptr()), n));  // gpu_relu
	auto in = input.get_smart_ptr();
	result.get_smart_ptr()->children = { in };  // l-ten/layers.cpp:61-63
	result.get_smart_ptr()->autograd = true;
	result.get_smart_ptr()->grad_fn = [in, n](TensorImpl&, const float* top) {
		if (!wants_gradient(in)) return;
		Bottom g(in);
		if (g.temporary) {  // l-ten/backprop.cpp:2282-2327: bottom = input > 0 ? top : 0
			LTEN_HIP_CALL(lten_hip_relu_backward_f32(g.ptr, top, static_cast<const float*>(in->data), n));
		} else {  // a leaf accumulates (l-ten/backprop.cpp:246-274)
			float* tmp = static_cast<float*>(TensorImpl::alloc(GPU, n * sizeof(float), false));
			LTEN_HIP_CALL(lten_hip_relu_backward_f32(tmp, top, static_cast<const float*>(in->data), n));
			LTEN_HIP_CALL(lten_hip_axpy_f32(n, 1.0f, tmp, g.ptr));
			LTEN_HIP_CALL(lten_hip_sync());
			TensorImpl::release(GPU, tmp);
		}
		g.propagate();
	};
	return result;
}

Tensor log_softmax(Tensor& input, int dim)
{
	require_gpu_f32(input, "log_softmax");
	const int ndims = input.get_ndims();
	if (dim != ndims - 1) LTEN_ERR("this build implements log_softmax along the last dimension only");
	const uint64_t cols = input.get_sizes()[ndims - 1], rows = cols ? input.get_numels() / cols : 0;
	TensorOps options;
	options.device_index = input.get_device_index();
	options.device_type = GPU;
	Tensor result = AllocateTensor(input.get_sizes(), ndims, &options);
	LTEN_HIP_CALL(lten_hip_log_softmax_f32(rows, cols, static_cast<const float*>(input.get_data_ptr()), static_cast<float*>(result.get_data_ptr())));
	auto in = input.get_smart_ptr(), out = result.get_smart_ptr();
	TensorImpl* out_raw = out.get();  // the node owns the closure: no shared_ptr cycle
	result.get_smart_ptr()->children = { in };
	result.get_smart_ptr()->autograd = true;
	result.get_smart_ptr()->grad_fn = [in, out_raw, rows, cols](TensorImpl&, const float* top) {
		if (!wants_gradient(in)) return;
		Bottom g(in);
		const uint64_t n = rows * cols;
		float* tmp = g.temporary ? g.ptr : static_cast<float*>(TensorImpl::alloc(GPU, n * sizeof(float), false));
		// l-ten's backward functions of log, div, sum, exp, sub and max add up to dy - exp(y) * sum_j dy_j
		LTEN_HIP_CALL(lten_hip_log_softmax_backward_f32(rows, cols, static_cast<const float*>(out_raw->data), top, tmp));
		if (!g.temporary) {
			LTEN_HIP_CALL(lten_hip_axpy_f32(n, 1.0f, tmp, g.ptr));
			LTEN_HIP_CALL(lten_hip_sync());
			TensorImpl::release(GPU, tmp);
		}
		g.propagate();
	};
	return result;
}

Tensor nll_loss(Tensor& input, Tensor& target)
{
	require_gpu_f32(input, "nll_loss");
	require_gpu_f32(target, "nll_loss");
	if (input.get_numels() != target.get_numels()) LTEN_ERR("nll_loss: input and target must have the same number of elements");
	TensorOps options;
	options.device_index = input.get_device_index();
	options.device_type = GPU;
	Tensor result = AllocateTensor({ 1 }, &options);  // l-ten/layers.cpp:231-232
	const uint64_t len = input.get_numels(), batch = input.get_sizes()[0];
	LTEN_HIP_CALL(lten_hip_nll_loss_f32(static_cast<const float*>(input.get_data_ptr()), static_cast<const float*>(target.get_data_ptr()),
	                                    static_cast<float*>(result.get_data_ptr()), len, batch));  // gpu_nll, :254
	auto in = input.get_smart_ptr(), tg = target.get_smart_ptr();
	result.get_smart_ptr()->children = { in, tg };  // :266-269
	result.get_smart_ptr()->autograd = true;
	result.get_smart_ptr()->grad_fn = [in, tg, len, batch](TensorImpl&, const float* top) {
		// l-ten/backprop.cpp:3975-4040: scale = -1 / batch * top[0]; bottom = scale * (the other operand)
		float top_value = 1.0f;
		LTEN_HIP_CALL(lten_hip_copy_from_gpu(&top_value, top, sizeof(float)));
		const float scale = (-1.0f / (float)batch) * top_value;
		const std::shared_ptr<TensorImpl> pair[2][2] = { { in, tg }, { tg, in } };
		for (auto& p : pair) {
			if (!wants_gradient(p[0])) continue;
			Bottom g(p[0]);
			if (g.temporary) LTEN_HIP_CALL(lten_hip_scale_f32(len, scale, static_cast<const float*>(p[1]->data), g.ptr));
			else LTEN_HIP_CALL(lten_hip_axpy_f32(len, scale, static_cast<const float*>(p[1]->data), g.ptr));
			g.propagate();
		}
	};
	return result;
}

// ------------------------------------------------------------------------------ FullyConnected_q

bool FullyConnected_q::init()
{
	// l-ten/fully_connected.cpp:295-320: UINT8 weights {1,1,out,in}, INT32 bias {out}, no initialisation
	TensorOps options;
	options.data_type = UINT8;
	weight_ = AllocateTensor({ 1, 1, output_features_, input_features_ }, &options);
	weight_.set_autograd(true);
	if (use_bias_) {
		options.data_type = INT32;
		bias_ = AllocateTensor({ output_features_ }, &options);
		bias_.set_autograd(true);
	}
	return true;
}

void FullyConnected_q::to(device target_device, int target_device_index)
{
	// l-ten's FullyConnected_q::to throws "Only CPU device supported" (l-ten/layers.h:86); this is the GPU branch it lacks
	if (weight_.defined()) weight_ = weight_.to(target_device, target_device_index);
	if (use_bias_ && bias_.defined()) bias_ = bias_.to(target_device, target_device_index);
	workspace_ = Tensor();
	max_rows_ = 0;
	prepared_ = Tensor();  // the int8 copy of the weights and their row sums are made again by the next forward
	weight_sums_ = Tensor();
	prepared_valid_ = false;
}

void FullyConnected_q::clear_gradients()
{
	if (weight_.defined()) weight_.clear_gradients();
	if (use_bias_ && bias_.defined()) bias_.clear_gradients();
}

std::vector<Tensor*> FullyConnected_q::get_all_weights()
{
	prepared_valid_ = false;  // the caller may write new weights through these (l-ten/net.h:227-236 does)
	std::vector<Tensor*> w{ &weight_ };
	if (use_bias_) w.push_back(&bias_);
	return w;
}

void FullyConnected_q::set_qparams_params(QuantizationParams* qparams, int count)
{
	if (qparams && count) qparams_wt_ = qparams[0];  // l-ten/fully_connected.cpp:440-446
}

Tensor FullyConnected_q::forward(Tensor& input)
{
	const int ndims = input.get_ndims();
	if (ndims < 3) LTEN_ERR("FullyConnected_q requires tensors with at least 3 dimensions");  // l-ten/fully_connected.cpp:331-334
	check_layer_input(input, weight_, "FullyConnected_q");
	uint64_t dims[MAX_DIMS];
	memcpy(dims, input.get_sizes(), sizeof(uint64_t) * ndims);
	if (dims[ndims - 1] != input_features_) LTEN_ERR("Last dimension must be equal to the number of input features");
	dims[ndims - 1] = output_features_;
	if (input.get_device() != GPU)
		LTEN_ERR("this build implements FullyConnected_q for the GPU device type only (l-ten's own CPU path covers lten::CPU)");

	TensorOps options;
	options.data_type = UINT8;
	options.device_index = input.get_device_index();
	options.device_type = GPU;
	Tensor result = AllocateTensor(dims, ndims, &options);
	// l-ten/fully_connected.cpp:364-396 loops one quantized_matmul over the leading dims with M = dims[ndims-2];
	// the rows are independent, so the loop is one call with batch * M rows
	const uint64_t M = dims[ndims - 2];
	uint64_t batch = 1;
	for (int i = 0; i < ndims - 2; i++) batch *= dims[i];
	if (batch * M > max_rows_) {  // :366-371 workspace grown on demand
		options.data_type = INT32;
		workspace_ = AllocateTensor({ batch * M + output_features_ }, &options);
		max_rows_ = batch * M;
	}
	lten_hip_qparams qp[3] = { { qparams_in_.scale, qparams_in_.zero_point }, { qparams_wt_.scale, qparams_wt_.zero_point },
		                   { qparams_out_.scale, qparams_out_.zero_point } };
	// The weights are constant between forward calls: their int8 form (w - 128, what the matrix cores multiply) and the
	// byte sum of every weight row (the zero-point correction's column term, l-ten/math_fns.cpp:1362-1369) are made
	// once per to() / weights_changed() / hand-out of the weight tensor, and every forward runs on them.
	if (!prepared_valid_) {
		options.data_type = UINT8;
		// (rows of the int8 form start on 16-byte boundaries: input_features_ rounded up to a multiple of 16 bytes apart)
		if (!prepared_.defined()) prepared_ = AllocateTensor({ 1, 1, output_features_, (input_features_ + 15) / 16 * 16 }, &options);
		options.data_type = INT32;
		if (!weight_sums_.defined()) weight_sums_ = AllocateTensor({ output_features_ }, &options);
		LTEN_HIP_CALL(lten_hip_fcq_prepare_weights(static_cast<const uint8_t*>(weight_.get_data_ptr()), static_cast<uint8_t*>(prepared_.get_data_ptr()),
		                                           output_features_, input_features_, static_cast<int32_t*>(weight_sums_.get_data_ptr())));
		prepared_valid_ = true;
	}
	LTEN_HIP_CALL(lten_hip_fcq_forward_prepared(batch, M, input_features_, output_features_, static_cast<const uint8_t*>(input.get_data_ptr()),
	                                            static_cast<const uint8_t*>(prepared_.get_data_ptr()),
	                                            static_cast<const int32_t*>(weight_sums_.get_data_ptr()),
	                                            use_bias_ ? static_cast<const int32_t*>(bias_.get_data_ptr()) : nullptr, qp,
	                                            static_cast<uint8_t*>(result.get_data_ptr()), static_cast<int32_t*>(workspace_.get_data_ptr())));
	return result;
}

// ------------------------------------------------------------------------------ Conv2d

bool Conv2d::init()
{
	// l-ten/conv2d.cpp:10-53: weight {Cout, Cin, kh*kw}, bias {1,Cout,1,1}, U(+-sqrt(1/(Cin*(kh+kw)))) from a default-seeded engine
	TensorOps options;
	weight_ = AllocateTensor({ channels_out_, channels_in_, kernel_h_ * kernel_w_ }, &options);
	weight_.set_autograd(true);
	std::default_random_engine generator;
	const float k = 1.0f / (channels_in_ * (kernel_h_ + kernel_w_));
	std::uniform_real_distribution<float> distribution(-sqrtf(k), sqrtf(k));
	float* w = static_cast<float*>(weight_.get_data_ptr());
	for (uint64_t i = 0; i < weight_.get_numels(); i++) w[i] = distribution(generator);
	if (use_bias_) {
		bias_ = AllocateTensor({ 1, channels_out_, 1, 1 }, &options);
		bias_.set_autograd(true);
		float* b = static_cast<float*>(bias_.get_data_ptr());
		for (uint64_t i = 0; i < bias_.get_numels(); i++) b[i] = distribution(generator);
	}
	return true;
}

void Conv2d::to(device target_device, int target_device_index)
{
	if (weight_.defined()) weight_ = weight_.to(target_device, target_device_index);
	if (use_bias_ && bias_.defined()) bias_ = bias_.to(target_device, target_device_index);
	scratch_ = Tensor();
}

void Conv2d::clear_gradients()
{
	if (weight_.defined()) weight_.clear_gradients();
	if (use_bias_ && bias_.defined()) bias_.clear_gradients();
}

std::vector<Tensor*> Conv2d::get_all_weights()
{
	std::vector<Tensor*> w{ &weight_ };
	if (use_bias_) w.push_back(&bias_);
	return w;
}


Tensor Conv2d::forward(Tensor& input)
{
	if (input.get_data_type() != FLOAT32) LTEN_ERR("Conv2d is only supported for FLOAT32 tensors");  // l-ten/conv2d.cpp:73-76
	check_layer_input(input, weight_, "Conv2d");
	if (input.get_ndims() != 4) LTEN_ERR("Conv2d requires tensors with exactly 4 dimensions (NCHW)");  // :86-89
	const uint64_t* d = input.get_sizes();
	const uint64_t N = d[0], H = d[2], W = d[3];
	if (d[1] != channels_in_) LTEN_ERR("Input channel count does not match this layer");
	const uint64_t Ho = (H + 2 * pad_h_ - kernel_h_) / stride_h_ + 1, Wo = (W + 2 * pad_w_ - kernel_w_) / stride_w_ + 1;  // :102-103
	if (input.get_device() != GPU)
		LTEN_ERR("this build implements Conv2d for the GPU device type only (l-ten's own CPU path covers lten::CPU)");

	TensorOps options;
	options.device_index = input.get_device_index();
	options.device_type = GPU;
	Tensor result = AllocateTensor({ N, channels_out_, Ho, Wo }, &options);
	const uint64_t Cin = channels_in_, Cout = channels_out_;
	const int kh = (int)kernel_h_, kw = (int)kernel_w_, ph = (int)pad_h_, pw = (int)pad_w_, sh = (int)stride_h_, sw = (int)stride_w_;
	// l-ten/conv2d.cpp:164-171 (im2col_gpu + cublasSgemm per image) and :189-192 (bias as a broadcast add): one fused launch
	LTEN_HIP_CALL(lten_hip_conv2d_forward_f32(N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, static_cast<const float*>(input.get_data_ptr()),
	                                          static_cast<const float*>(weight_.get_data_ptr()),
	                                          use_bias_ ? static_cast<const float*>(bias_.get_data_ptr()) : nullptr,
	                                          static_cast<float*>(result.get_data_ptr())));

	// scratch: [workspace of the weight / data gradient calls, whichever is larger][temp dW][temp dX for a whole batch]
	const uint64_t Kc = Cin * kernel_h_ * kernel_w_;
	const uint64_t ws_bytes = std::max(lten_hip_conv2d_wgrad_workspace_bytes(N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw),
	                                   lten_hip_conv2d_dgrad_workspace_bytes(N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw));
	const uint64_t work_floats = (ws_bytes + 3) / 4 + 64;
	const uint64_t need = work_floats + Cout * Kc + N * Cin * H * W;
	if (!scratch_.defined() || scratch_.get_numels() < need) scratch_ = AllocateTensor({ need }, &options);
	auto wt = weight_.get_smart_ptr(), in = input.get_smart_ptr(), scratch = scratch_.get_smart_ptr();
	const bool with_bias = use_bias_;
	auto bs = use_bias_ ? bias_.get_smart_ptr() : std::shared_ptr<TensorImpl>();
	result.get_smart_ptr()->children = { wt, in };  // l-ten/conv2d.cpp:183-187
	result.get_smart_ptr()->autograd = true;
	result.get_smart_ptr()->grad_fn = [=](TensorImpl&, const float* top) {
		if (with_bias && wants_gradient(bs)) {
			// l-ten/conv2d.cpp:189-192 adds the bias as a broadcast tensor op; its backward pass (l-ten/backprop.cpp:605-690)
			// sums the top gradient over N, H, W into the bias gradient
			bs->ensure_grad();
			LTEN_HIP_CALL(lten_hip_conv2d_bias_grad_f32(N, Cout, (uint64_t)Ho * Wo, top, static_cast<float*>(bs->grad), 1));
		}
		float* work = static_cast<float*>(scratch->data);
		float* tmp_dw = work + work_floats;
		float* tmp_dx = tmp_dw + Cout * Kc;
		const float* x = static_cast<const float*>(in->data);
		const float* w = static_cast<const float*>(wt->data);
		if (wants_gradient(wt)) {
			// l-ten/backprop.cpp:1949-1953 (CPU semantics: the sum over all images), then the leaf accumulate of :246-274
			Bottom g(wt);
			LTEN_HIP_CALL(lten_hip_conv2d_wgrad_f32(N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, x, top, tmp_dw, work));
			LTEN_HIP_CALL(lten_hip_axpy_f32(Cout * Kc, 1.0f, tmp_dw, g.ptr));
		}
		if (wants_gradient(in)) {
			// l-ten/backprop.cpp:2022-2028 (per image col = W^T dY_n, then col2im) for the whole batch, then the accumulate
			Bottom g(in);
			LTEN_HIP_CALL(lten_hip_conv2d_dgrad_f32(N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, w, top, tmp_dx, work));
			LTEN_HIP_CALL(lten_hip_axpy_f32(N * Cin * H * W, 1.0f, tmp_dx, g.ptr));
			g.propagate();
		}
	};
	return result;
}

// ------------------------------------------------------------------------------ Conv2d_q

bool Conv2d_q::init()
{
	// l-ten/conv2d.cpp:235-263: UINT8 weights {Cout, Cin, kh*kw}, INT32 bias {1,Cout,1,1}, no initialisation
	TensorOps options;
	options.data_type = UINT8;
	weight_ = AllocateTensor({ channels_out_, channels_in_, kernel_h_ * kernel_w_ }, &options);
	weight_.set_autograd(true);
	if (use_bias_) {
		options.data_type = INT32;
		bias_ = AllocateTensor({ 1, channels_out_, 1, 1 }, &options);
		bias_.set_autograd(true);
	}
	return true;
}

void Conv2d_q::to(device target_device, int target_device_index)
{
	// l-ten's Conv2d_q::to throws "Only CPU device supported" (l-ten/layers.h:498); this is the GPU branch it lacks
	if (weight_.defined()) weight_ = weight_.to(target_device, target_device_index);
	if (use_bias_ && bias_.defined()) bias_ = bias_.to(target_device, target_device_index);
	workspace_ = Tensor();
}

void Conv2d_q::clear_gradients()
{
	if (weight_.defined()) weight_.clear_gradients();
	if (use_bias_ && bias_.defined()) bias_.clear_gradients();
}

std::vector<Tensor*> Conv2d_q::get_all_weights()
{
	std::vector<Tensor*> w{ &weight_ };
	if (use_bias_) w.push_back(&bias_);
	return w;
}

void Conv2d_q::set_qparams_params(QuantizationParams* qparams, int count)
{
	if (qparams && count) qparams_wt_ = qparams[0];  // l-ten/conv2d.cpp:415-421
}

Tensor Conv2d_q::forward(Tensor& input)
{
	if (input.get_data_type() != UINT8) LTEN_ERR("Conv2d_q is only supported for UINT8 tensors");  // l-ten/conv2d.cpp:284-288
	check_layer_input(input, weight_, "Conv2d_q");
	if (input.get_ndims() != 4) LTEN_ERR("Conv2d_q requires tensors with exactly 4 dimensions (NCHW)");  // :299-302
	const uint64_t* d = input.get_sizes();
	const uint64_t N = d[0], H = d[2], W = d[3];
	if (d[1] != channels_in_) LTEN_ERR("Input channel count does not match this layer");
	const uint64_t Ho = (H + 2 * pad_h_ - kernel_h_) / stride_h_ + 1, Wo = (W + 2 * pad_w_ - kernel_w_) / stride_w_ + 1;  // :314-315
	if (input.get_device() != GPU)
		LTEN_ERR("this build implements Conv2d_q for the GPU device type only (l-ten's own CPU path covers lten::CPU)");
	// l-ten hands its Cout-element bias to quantized_matmul, which indexes it by output position (l-ten/conv2d.cpp:366,
	// l-ten/math_fns.cpp:1470-1473): with more output positions than channels that call reads past the buffer.
	if (use_bias_ && Ho * Wo > channels_out_)
		LTEN_ERR("Conv2d_q with a bias: l-ten's call indexes the bias by output position and would read past its Cout elements");

	TensorOps options;
	options.data_type = UINT8;
	options.device_index = input.get_device_index();
	options.device_type = GPU;
	Tensor result = AllocateTensor({ N, channels_out_, Ho, Wo }, &options);
	const int kh = (int)kernel_h_, kw = (int)kernel_w_, ph = (int)pad_h_, pw = (int)pad_w_, sh = (int)stride_h_, sw = (int)stride_w_;
	const uint64_t need = lten_hip_conv2dq_workspace_bytes(N, channels_in_, H, W, channels_out_, kh, kw, ph, pw, sh, sw);
	if (!workspace_.defined() || workspace_.get_numels() < need) workspace_ = AllocateTensor({ need }, &options);
	lten_hip_qparams qp[3] = { { qparams_in_.scale, qparams_in_.zero_point }, { qparams_wt_.scale, qparams_wt_.zero_point },
		                   { qparams_out_.scale, qparams_out_.zero_point } };
	// l-ten/conv2d.cpp:355-372 (im2col_cpu + quantized_matmul per image): one call for the batch
	LTEN_HIP_CALL(lten_hip_conv2dq_forward(N, channels_in_, H, W, channels_out_, kh, kw, ph, pw, sh, sw,
	                                       static_cast<const uint8_t*>(input.get_data_ptr()), static_cast<const uint8_t*>(weight_.get_data_ptr()),
	                                       use_bias_ ? static_cast<const int32_t*>(bias_.get_data_ptr()) : nullptr, qp,
	                                       static_cast<uint8_t*>(result.get_data_ptr()), workspace_.get_data_ptr()));
	return result;
}

// ---------------------------------------------------------------------------------------------------------
// NeuralNetwork and the optimizers (l-ten/net.h, l-ten/optimizer.{h,cpp})

NeuralNetwork::~NeuralNetwork()
{
	for (auto& p : params_) delete p.param_data_;
	for (Module* m : modules_) delete m;
}

NetworkParms* NeuralNetwork::get_parameters(int* num_params_ptr)
{
	if (!num_params_ptr) return nullptr;
	*num_params_ptr = (int)params_.size();
	return params_.data();
}

void NeuralNetwork::to(device target_device, int target_device_index)
{
	for (Module* m : modules_) m->to(target_device, target_device_index);
	for (auto& p : params_)
		if (p.param_data_) *p.param_data_ = p.param_data_->to(target_device, target_device_index);
}

void NeuralNetwork::train(bool is_training)
{
	for (Module* m : modules_) m->train(is_training);
}

Module* NeuralNetwork::get_module(int index)
{
	return index >= 0 && index < (int)modules_.size() ? modules_[index] : nullptr;
}

void Optimizer::attach_network(NeuralNetwork& net)
{
	network_params_ptr_ = net.get_parameters(&num_params_);
	setup_optimizer();
}

void Optimizer::zero_grad()
{
	for (int i = 0; i < num_params_; i++) network_params_ptr_[i].param_->clear_gradients();
}

Tensor* Optimizer::make_state(int param_index, uint64_t copies)
{
	Tensor* param = network_params_ptr_[param_index].param_;
	uint64_t dims[MAX_DIMS];
	memcpy(dims, param->get_sizes(), sizeof(uint64_t) * param->get_ndims());
	dims[0] *= copies;
	Tensor* state = new Tensor;
	*state = AllocateTensor(dims, param->get_ndims(), nullptr);
	memset(state->get_data_ptr(), 0, sizeof(float) * state->get_numels());
	if (param->get_device() == GPU) *state = state->to(GPU, param->get_device_index());
	return state;
}

void SGDOptimizer::setup_optimizer()
{
	for (int i = 0; i < num_params_; i++) {
		delete network_params_ptr_[i].param_data_;
		network_params_ptr_[i].param_data_ = make_state(i, 1);  // velocity
	}
}

void SGDOptimizer::step()
{
	if (!num_params_) LTEN_ERR("No parameters have been added to the optimizer");
	for (int i = 0; i < num_params_; i++) {
		Tensor* param = network_params_ptr_[i].param_;
		float* w = (float*)param->get_data_ptr();
		float* g = (float*)param->get_grad_ptr();
		float* v = (float*)network_params_ptr_[i].param_data_->get_data_ptr();
		const uint64_t numels = param->get_numels();
		if (!g) continue;  // a parameter that took no part in the last backward pass
		if (param->get_device() != network_params_ptr_[i].param_data_->get_device()) LTEN_ERR("Optimizer state and parameter are on different devices");
		if (param->get_device() == GPU) {
			LTEN_HIP_CALL(lten_hip_sgd_step_f32(w, g, v, numels, mo_, wd_, lr_));  // l-ten/optimizer.cpp:66
		} else {
			for (uint64_t j = 0; j < numels; j++) {  // l-ten/optimizer.cpp:49-54
				g[j] = wd_ * w[j] + g[j];
				v[j] = v[j] * mo_ + (1.0f - mo_) * g[j];
				w[j] = w[j] - (v[j] * lr_);
			}
		}
	}
}

void AdamOptimizer::setup_optimizer()
{
	for (int i = 0; i < num_params_; i++) {
		delete network_params_ptr_[i].param_data_;
		network_params_ptr_[i].param_data_ = make_state(i, 3);  // first moments, second moments, l-ten's scratch third
	}
}

void AdamOptimizer::step()
{
	if (!num_params_) LTEN_ERR("No parameters have been added to the optimizer");
	iteration_++;
	for (int i = 0; i < num_params_; i++) {
		Tensor* param = network_params_ptr_[i].param_;
		float* w = (float*)param->get_data_ptr();
		const float* g = (const float*)param->get_grad_ptr();
		const uint64_t numels = param->get_numels();
		float* v_dw = (float*)network_params_ptr_[i].param_data_->get_data_ptr();
		float* s_dw = v_dw + numels;
		if (!g) continue;
		if (param->get_device() != network_params_ptr_[i].param_data_->get_device()) LTEN_ERR("Optimizer state and parameter are on different devices");
		if (param->get_device() == GPU) {
			LTEN_HIP_CALL(lten_hip_adam_step_f32(w, g, v_dw, s_dw, numels, lr_, beta1_, beta2_, iteration_));  // l-ten/optimizer.cpp:165-172
		} else {
			// l-ten/optimizer.cpp:146-158, the eight element-wise passes in their order
			const float epsilon = 1.0e-8f;
			const float bc1 = 1.0f - powf(beta1_, (float)iteration_), bc2 = 1.0f - powf(beta2_, (float)iteration_);
			for (uint64_t j = 0; j < numels; j++) {
				v_dw[j] = (1.0f - beta1_) * g[j] + beta1_ * v_dw[j];
				s_dw[j] = (1.0f - beta2_) * (g[j] * g[j]) + beta2_ * s_dw[j];
				float t = (1.0f / bc2) * s_dw[j];
				t = powf(t, 0.5f) + epsilon;
				t = v_dw[j] / t;
				w[j] = -(1.0f / bc1) * lr_ * t + w[j];
			}
		}
	}
}

}  // namespace lten
