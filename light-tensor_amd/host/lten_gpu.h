// Host-side mirror of l-ten's layer API for the GEMM hot path, over the C ABI of liblten_hip.
//
// Same names, argument meaning and error behaviour as l-ten's lten::Tensor / FullyConnected /
// FullyConnected_q / Conv2d / Tensor::matmul (l-ten/tensor.h, l-ten/layers.h), reduced to what the hot
// path needs.  It is the shape of the glue a maintainer adds to l-ten's own `#ifdef USE_CUDA` branches:
// every GPU branch below is one call through include/lten_hip.h.  Tensors on lten::CPU only carry data
// in and out (TensorFromBuffer, to()); the arithmetic itself exists for lten::GPU tensors only — there
// is no CPU compute path in this library, l-ten already has one.
#ifndef LTEN_GPU_H
#define LTEN_GPU_H

#include <cstdint>
#include <exception>
#include <functional>
#include <initializer_list>
#include <memory>
#include <string>
#include <vector>

// l-ten/md_array.h:37
#define MAX_DIMS 16

// l-ten/math_fns.h:12-16 (global namespace there too)
struct QuantizationParams {
	float scale;
	uint8_t zero_point;
};

namespace lten {

// l-ten/tensorimpl.h:46-47
enum device { CPU, GPU };
enum dtype { FLOAT32, INT32, UINT8 };

// l-ten/tensorimpl.h:49-63
struct TensorOps {
	TensorOps() : data_type(FLOAT32), device_type(CPU), device_index(0), alloc_gradient_buffer(false) {}
	dtype data_type;
	device device_type;
	int device_index;
	bool alloc_gradient_buffer;
};

// What LTEN_ERR throws (l-ten/error.h:78-93, l-ten/utils.cpp:303-306).
class ExceptionInfo : public std::exception {
public:
	ExceptionInfo(const char* msg, const char* file, const char* func, int line);
	const char* what() const noexcept override { return text_.c_str(); }

private:
	std::string text_;
};
[[noreturn]] void ltenFail(const char* msg, const char* file, const char* func, int line);
#define LTEN_ERR(msg) ::lten::ltenFail(msg, __FILE__, __func__, __LINE__)

struct TensorImpl;
class Tensor;
// gradient callback: (node, gradient of the loss with respect to the node's output on the node's device)
typedef std::function<void(TensorImpl& node, const float* top_gradient)> grad_fn_t;

class Tensor {
public:
	Tensor() {}
	explicit Tensor(std::shared_ptr<TensorImpl> impl) : impl_(impl) {}

	void* get_data_ptr();
	void* get_grad_ptr();
	uint64_t get_numels() const;
	const uint64_t* get_sizes() const;
	int get_ndims() const;
	dtype get_data_type() const;
	device get_device() const;
	int get_device_index() const;
	void set_autograd(bool setting);
	void clear_gradients();

	// l-ten/tensor.h:140-..., l-ten/tensorimpl.cpp:311-412: copy to the other device (synchronous).
	Tensor to(device target_device, int target_device_index = 0);
	// l-ten/tensor.h:83-138: batched matrix product over the leading dims, size-1 dims broadcast.
	Tensor matmul(const Tensor& other);
	// l-ten/tensor.h:1152-1200, l-ten/tensorimpl.cpp:2033-2052: the same buffer under other dimensions (same element
	// count); the source stays alive as the result's child and receives the result's gradient unchanged.
	Tensor reshape(const std::initializer_list<uint64_t>& dims);
	// l-ten/tensor.h:69 backward(MultiDimArray<float>* top_gradient): top_gradient has the tensor's shape and
	// lives on the tensor's device; null stands for a single 1 and is only valid for one-element tensors.
	void backward(const Tensor* top_gradient = nullptr);

	std::shared_ptr<TensorImpl> get_smart_ptr() const { return impl_; }
	bool defined() const { return impl_ != nullptr; }

private:
	std::shared_ptr<TensorImpl> impl_;
};

// l-ten/tensor.h:1478-1482
Tensor TensorFromBuffer(const std::initializer_list<uint64_t>& dims, void* data_ptr, bool own_memory = false, TensorOps* options_ptr = nullptr);
Tensor TensorFromBuffer(const uint64_t* dims_ptr, int ndims, void* data_ptr, bool own_memory = false, TensorOps* options_ptr = nullptr);
Tensor AllocateTensor(const std::initializer_list<uint64_t>& dims, TensorOps* options_ptr = nullptr);
Tensor AllocateTensor(const uint64_t* dims_ptr, int ndims, TensorOps* options_ptr = nullptr);

// l-ten/layers.h (free functions): the element-wise and loss pieces of a training step, GPU tensors only.
Tensor relu(Tensor& input);                        // l-ten/layers.cpp:9-67
Tensor log_softmax(Tensor& input, int dim);        // l-ten/layers.cpp:93-114; dim must be the last dimension here
Tensor nll_loss(Tensor& input, Tensor& target);    // l-ten/layers.cpp:212-273

// l-ten/layers.h:14-31
class Module {
public:
	Module() {}
	virtual ~Module() {}
	virtual bool init() = 0;
	virtual std::vector<Tensor*> get_all_weights() = 0;
	virtual void clear_gradients() = 0;
	virtual void to(device target_device, int target_device_index = 0) = 0;
	void train(bool is_training) { is_training_ = is_training; }
	virtual void set_qparams_in(QuantizationParams) {}
	virtual void set_qparams_out(QuantizationParams) {}
	virtual void set_qparams_params(QuantizationParams*, int) {}

protected:
	bool is_training_ = true;
};

// l-ten/layers.h:35-66
class FullyConnected : public Module {
public:
	FullyConnected(int64_t input_features, int64_t output_features, bool use_bias = false, dtype data_type = FLOAT32)
	    : input_features_(input_features), output_features_(output_features), use_bias_(use_bias) { (void)data_type; }
	bool init() override;
	Tensor forward(Tensor& input);
	Tensor* get_weights() { return &weight_; }
	Tensor* get_bias() { return use_bias_ ? &bias_ : nullptr; }
	void clear_gradients() override;
	std::vector<Tensor*> get_all_weights() override;
	void to(device target_device, int target_device_index = 0) override;
	bool is_using_bias() { return use_bias_; }

private:
	uint64_t input_features_, output_features_;
	Tensor weight_, bias_;
	bool use_bias_;
};

// l-ten/layers.h:69-106; unlike l-ten's, this one runs on the GPU (l-ten: "Only CPU device supported").
class FullyConnected_q : public Module {
public:
	FullyConnected_q(int64_t input_features, int64_t output_features, bool use_bias = false, dtype data_type = FLOAT32)
	    : input_features_(input_features), output_features_(output_features), use_bias_(use_bias) { (void)data_type; }
	bool init() override;
	Tensor forward(Tensor& input);
	// The accessors that hand out the weight tensor for writing (l-ten's load_checkpoint fills GPU-resident parameters
	// through get_all_weights, l-ten/net.h:227-236) mark the layer's int8 copy of the weights stale: the next forward
	// converts them again.  A caller that keeps the pointer and writes through it after a later forward must call
	// weights_changed() itself.
	Tensor* get_weights() { prepared_valid_ = false; return &weight_; }
	Tensor* get_bias() { return use_bias_ ? &bias_ : nullptr; }
	void clear_gradients() override;
	std::vector<Tensor*> get_all_weights() override;
	void to(device target_device, int target_device_index = 0) override;
	bool is_using_bias() { return use_bias_; }
	void set_qparams_in(QuantizationParams qparams_in) override { qparams_in_ = qparams_in; }
	void set_qparams_out(QuantizationParams qparams_out) override { qparams_out_ = qparams_out; }
	void set_qparams_params(QuantizationParams* qparams, int count) override;
	// to be called after writing new weight bytes into get_weights() while the layer is on the GPU (to() does it itself)
	void weights_changed() { prepared_valid_ = false; }

private:
	uint64_t input_features_, output_features_;
	Tensor weight_, bias_, workspace_;
	Tensor prepared_;     // int8 form of weight_ for the GEMM (lten_hip_fcq_prepare_weights)
	Tensor weight_sums_;  // byte sum of every weight row, made by the same call
	bool prepared_valid_ = false;
	bool use_bias_;
	uint64_t max_rows_ = 0;
	QuantizationParams qparams_in_{ 1.0f, 0 }, qparams_out_{ 1.0f, 0 }, qparams_wt_{ 1.0f, 0 };
};

// l-ten/layers.h:392-451
class Conv2d : public Module {
public:
	Conv2d(const int channels_in, const int channels_out, bool use_bias, const int kernel_h, const int kernel_w, const int pad_h = 0,
	       const int pad_w = 0, const int stride_h = 1, const int stride_w = 1)
	    : channels_in_(channels_in), channels_out_(channels_out), kernel_h_(kernel_h), kernel_w_(kernel_w), pad_h_(pad_h), pad_w_(pad_w),
	      stride_h_(stride_h), stride_w_(stride_w), use_bias_(use_bias) {}
	uint64_t get_channels_out() { return channels_out_; }
	uint64_t get_channels_in() { return channels_in_; }
	uint64_t get_kernel_h() { return kernel_h_; }
	uint64_t get_kernel_w() { return kernel_w_; }
	uint64_t get_pad_h() { return pad_h_; }
	uint64_t get_pad_w() { return pad_w_; }
	uint64_t get_stride_h() { return stride_h_; }
	uint64_t get_stride_w() { return stride_w_; }
	bool init() override;
	Tensor forward(Tensor& input);
	std::vector<Tensor*> get_all_weights() override;
	Tensor* get_weights() { return &weight_; }
	Tensor* get_bias() { return use_bias_ ? &bias_ : nullptr; }
	void clear_gradients() override;
	void to(device target_device, int target_device_index = 0) override;

private:
	uint64_t channels_in_, channels_out_, kernel_h_, kernel_w_, pad_h_, pad_w_, stride_h_, stride_w_;
	bool use_bias_;
	Tensor weight_, bias_, scratch_;  // scratch_: weight-gradient partial sums / column buffer of the data gradient
};

// l-ten/layers.h:453-524; unlike l-ten's, this one runs on the GPU (l-ten: "Only CPU device supported").  Inference only,
// as in l-ten (the result carries no usable gradient function for uint8 data).
class Conv2d_q : public Module {
public:
	Conv2d_q(const int channels_in, const int channels_out, bool use_bias, const int kernel_h, const int kernel_w, const int pad_h = 0,
	         const int pad_w = 0, const int stride_h = 1, const int stride_w = 1)
	    : channels_in_(channels_in), channels_out_(channels_out), kernel_h_(kernel_h), kernel_w_(kernel_w), pad_h_(pad_h), pad_w_(pad_w),
	      stride_h_(stride_h), stride_w_(stride_w), use_bias_(use_bias) {}
	uint64_t get_channels_out() { return channels_out_; }
	uint64_t get_channels_in() { return channels_in_; }
	uint64_t get_kernel_h() { return kernel_h_; }
	uint64_t get_kernel_w() { return kernel_w_; }
	uint64_t get_pad_h() { return pad_h_; }
	uint64_t get_pad_w() { return pad_w_; }
	uint64_t get_stride_h() { return stride_h_; }
	uint64_t get_stride_w() { return stride_w_; }
	bool init() override;
	Tensor forward(Tensor& input);
	std::vector<Tensor*> get_all_weights() override;
	Tensor* get_weights() { return &weight_; }
	Tensor* get_bias() { return use_bias_ ? &bias_ : nullptr; }
	void clear_gradients() override;
	void to(device target_device, int target_device_index = 0) override;
	void set_qparams_in(QuantizationParams qparams_in) override { qparams_in_ = qparams_in; }
	void set_qparams_out(QuantizationParams qparams_out) override { qparams_out_ = qparams_out; }
	void set_qparams_params(QuantizationParams* qparams, int count) override;

private:
	uint64_t channels_in_, channels_out_, kernel_h_, kernel_w_, pad_h_, pad_w_, stride_h_, stride_w_;
	bool use_bias_;
	Tensor weight_, bias_, workspace_;
	QuantizationParams qparams_in_{ 1.0f, 0 }, qparams_out_{ 1.0f, 0 }, qparams_wt_{ 1.0f, 0 };
};

// l-ten/net.h:8-19
struct NetworkParms {
	std::string name;
	Tensor* param_;       // trainable parameter
	Tensor* param_data_;  // what an optimizer keeps for it (velocity, moment histories), or null
};

// l-ten/net.h:21-117: owns the modules registered with it and lists their trainable parameters for an optimizer.
// A network class derives from it and registers its layers in its constructor, as in l-ten.
class NeuralNetwork {
public:
	NeuralNetwork() {}
	NeuralNetwork(const NeuralNetwork&) = delete;
	NeuralNetwork& operator=(const NeuralNetwork&) = delete;
	~NeuralNetwork();

	template <typename T>
	T* register_module(const char* module_name, T&& temp)
	{
		T* network_module = new T(temp);
		network_module->init();
		for (Tensor* param : network_module->get_all_weights()) params_.push_back(NetworkParms{ module_name ? module_name : "", param, nullptr });
		modules_.push_back(network_module);
		return network_module;
	}
	NetworkParms* get_parameters(int* num_params_ptr);
	void to(device target_device, int target_device_index = 0);
	void train(bool is_training);
	Module* get_module(int index);

private:
	std::vector<NetworkParms> params_;
	std::vector<Module*> modules_;
};

// l-ten/optimizer.h:6-33.  The state tensors live where the parameters live when the network is attached and
// move with NeuralNetwork::to afterwards; l-ten allocates them on the CPU and relies on a later to().
class Optimizer {
public:
	Optimizer() {}
	virtual ~Optimizer() {}
	void attach_network(NeuralNetwork& net);
	virtual void setup_optimizer() = 0;
	virtual void step() = 0;
	void zero_grad();

protected:
	Tensor* make_state(int param_index, uint64_t copies);  // zero-filled, copies x the parameter's first dimension
	int num_params_ = 0;
	NetworkParms* network_params_ptr_ = nullptr;
};

// l-ten/optimizer.h:35-58, l-ten/optimizer.cpp:10-84
class SGDOptimizer : public Optimizer {
public:
	void setup_optimizer() override;
	void step() override;
	void set_learning_rate(float lr) { lr_ = lr; }
	float get_learning_rate() { return lr_; }
	void set_momentum(float mo) { mo_ = mo; }
	float get_momentum() { return mo_; }
	void set_weight_decay(float wd) { wd_ = wd; }
	float get_weight_decay() { return wd_; }

private:
	float lr_ = 0.01f, wd_ = 0.0005f, mo_ = 0.9f;
};

// l-ten/optimizer.h:60-84, l-ten/optimizer.cpp:88-186
class AdamOptimizer : public Optimizer {
public:
	void setup_optimizer() override;
	void step() override;
	void set_learning_rate(float lr) { lr_ = lr; }
	float get_learning_rate() { return lr_; }
	void set_beta1(float beta1) { beta1_ = beta1; }
	float get_beta1() { return beta1_; }
	void set_beta2(float beta2) { beta2_ = beta2; }
	float get_beta2() { return beta2_; }

private:
	uint64_t iteration_ = 0;
	float lr_ = 0.01f, beta1_ = 0.9f, beta2_ = 0.999f;
};

}  // namespace lten
#endif
