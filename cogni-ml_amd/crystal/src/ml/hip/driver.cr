# ML::HIP - Crystal binding of libcogni_hip.so for MI355X (gfx950).
#
# Mirrors src/ml/cuda/driver.cr class for class so runner code ports by renaming ML::CUDA -> ML::HIP:
# Context, DeviceBuffer, HIPModule (CUDAModule), KernelFunction, FunctionAttribute, HIPStream, HIPGraph,
# HIPGraphExec, with_stream, copy_htod!/dtoh!/dtod!, synchronize!, launch!, ResidentSequenceRunner.
# The `fun` declarations below are include/ml_hip_driver.h and the level-1/2 part of include/cogni_quant.h.
#
# NOT COMPILED in the environment this was written in (no Crystal compiler there); the same C entry points
# are exercised from C++ (cogni-ml_amd/host/ml_hip.hpp) and Python ctypes (cogni_ml_amd/hip.py).
@[Link(ldflags: "-lcogni_hip")]
lib LibCogniHIP
  alias Deviceptr = UInt64

  fun mlhip_init(flags : UInt32) : Int32
  fun mlhip_device_get(device : Int32*, ordinal : Int32) : Int32
  fun mlhip_device_get_name(name : UInt8*, len : Int32, dev : Int32) : Int32
  fun mlhip_device_compute_capability(major : Int32*, minor : Int32*, dev : Int32) : Int32
  fun mlhip_device_get_arch(name : UInt8*, len : Int32, dev : Int32) : Int32
  fun mlhip_ctx_create(ctx : Void**, flags : UInt32, dev : Int32) : Int32
  fun mlhip_ctx_destroy(ctx : Void*) : Int32
  fun mlhip_module_load_data(mod : Void**, image : Void*) : Int32
  fun mlhip_module_unload(mod : Void*) : Int32
  fun mlhip_module_get_function(fn : Void**, mod : Void*, name : UInt8*) : Int32
  fun mlhip_func_get_attribute(pi : Int32*, attrib : Int32, hfunc : Void*) : Int32
  fun mlhip_stream_create(stream : Void**, flags : UInt32) : Int32
  fun mlhip_stream_destroy(stream : Void*) : Int32
  fun mlhip_stream_synchronize(stream : Void*) : Int32
  fun mlhip_stream_begin_capture(stream : Void*, mode : Int32) : Int32
  fun mlhip_stream_end_capture(stream : Void*, graph : Void**) : Int32
  fun mlhip_graph_instantiate(exec : Void**, graph : Void*, flags : UInt64) : Int32
  fun mlhip_graph_upload(exec : Void*, stream : Void*) : Int32
  fun mlhip_graph_launch(exec : Void*, stream : Void*) : Int32
  fun mlhip_graph_destroy(graph : Void*) : Int32
  fun mlhip_graph_exec_destroy(exec : Void*) : Int32
  fun mlhip_mem_alloc(dptr : Deviceptr*, bytesize : LibC::SizeT) : Int32
  fun mlhip_mem_free(dptr : Deviceptr) : Int32
  fun mlhip_memcpy_htod(dst : Deviceptr, src : Void*, bytesize : LibC::SizeT) : Int32
  fun mlhip_memcpy_dtoh(dst : Void*, src : Deviceptr, bytesize : LibC::SizeT) : Int32
  fun mlhip_memcpy_dtod(dst : Deviceptr, src : Deviceptr, bytesize : LibC::SizeT) : Int32
  fun mlhip_launch_kernel(fn : Void*, grid_x : UInt32, grid_y : UInt32, grid_z : UInt32,
                          block_x : UInt32, block_y : UInt32, block_z : UInt32,
                          shared_mem_bytes : UInt32, stream : Void*,
                          kernel_params : Void**, extra : Void**) : Int32
  fun mlhip_ctx_synchronize : Int32
  fun mlhip_error_string(code : Int32) : UInt8*

  # include/cogni_quant.h
  fun cogni_quant_code_object(image : Void**, size : LibC::SizeT*) : Int32
  fun cogni_gemv_kernel_name(type : UInt32, tokens : UInt32, add : Int32) : UInt8*
  fun cogni_gemv_launch_dims(type : UInt32, tokens : UInt32, in_dim : UInt32, out_dim : UInt32,
                             grid_x : UInt32*, block_x : UInt32*, shared_mem_bytes : UInt32*) : Int32
  fun cogni_dequantize_kernel_name(type : UInt32) : UInt8*
  fun cogni_quant_init(ordinal : Int32) : Int32
  fun cogni_dequantize_dev(w_raw : UInt64, w_type : UInt32, n_elements : UInt64, out : UInt64, stream : Void*) : Int32
  fun cogni_gemv_dev(w_raw : UInt64, w_type : UInt32, x : UInt64, residual : UInt64, out : UInt64,
                     in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemv_plan(type : UInt32, tokens : UInt32, add : Int32, in_dim : UInt32, out_dim : UInt32, kernel : UInt8**,
                      grid_x : UInt32*, block_x : UInt32*, shared_mem_bytes : UInt32*) : Int32
  fun cogni_gemv_one_pass_from(w_type : UInt32, in_dim : UInt32, out_dim : UInt32) : UInt32
  fun cogni_gemv_one_pass_multi_from(w_type : UInt32, in_dim : UInt32) : UInt32
  fun cogni_gemv_passes(w_type : UInt32, tokens : UInt32, in_dim : UInt32, out_dim : UInt32) : Int32
  fun cogni_gemv_image_stats(slots : UInt32*, in_use : UInt32*, pinned : UInt32*, calls_without_image : UInt64*) : Int32
  fun cogni_gemv_release_stream(stream : Void*) : Int32
  fun cogni_gemv_image_bytes(w_type : UInt32, in_dim : UInt32, tokens : UInt32) : LibC::SizeT
  fun cogni_gemv_packed_launch_dims(w_type : UInt32, in_dim : UInt32, total_rows : UInt32,
                                    grid_x : UInt32*, block_x : UInt32*, shared_mem_bytes : UInt32*) : Int32
  fun cogni_gemv_pack_dev(x : UInt64, w_type : UInt32, in_dim : UInt32, tokens : UInt32, image : UInt64, stream : Void*) : Int32
  fun cogni_gemv_packed_dev(w_raw : UInt64*, w_type : UInt32, image : UInt64, residual : UInt64, out : UInt64*,
                            out_dims : UInt32*, count : UInt32, in_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemv_packed_swiglu_dev(w_gate : UInt64, w_up : UInt64, w_type : UInt32, image : UInt64, out : UInt64,
                                   in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemv_top1_noalloc_dev(w_raw : UInt64, w_type : UInt32, x : UInt64, top1_ids : UInt64, top1_values : UInt64,
                                  in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemv_dual_dev(w_raw_a : UInt64, w_raw_b : UInt64, w_type : UInt32, x : UInt64, out_a : UInt64, out_b : UInt64,
                          in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemv_many_dev(w_raw : UInt64*, w_type : UInt32, x : UInt64, out : UInt64*, out_dims : UInt32*, count : UInt32,
                          in_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_swiglu_dev(gate : UInt64, up : UInt64, out : UInt64, n : UInt32, stream : Void*) : Int32
  fun cogni_gemv_dual_swiglu_dev(w_gate : UInt64, w_up : UInt64, w_type : UInt32, x : UInt64, out : UInt64,
                                 in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_rmsnorm_dev(x : UInt64, norm : UInt64, out : UInt64, dim : UInt32, tokens : UInt32, eps : Float32,
                        stream : Void*) : Int32
  fun cogni_add_rmsnorm_dev(x : UInt64, add : UInt64, norm : UInt64, residual_out : UInt64, normed_out : UInt64,
                            dim : UInt32, tokens : UInt32, eps : Float32, stream : Void*) : Int32
  fun cogni_rmsnorm_pack_dev(x : UInt64, norm : UInt64, out : UInt64, w_type : UInt32, image : UInt64, dim : UInt32,
                             tokens : UInt32, eps : Float32, stream : Void*) : Int32
  fun cogni_add_rmsnorm_pack_dev(x : UInt64, add : UInt64, norm : UInt64, residual_out : UInt64, normed_out : UInt64,
                                 w_type : UInt32, image : UInt64, dim : UInt32, tokens : UInt32, eps : Float32,
                                 stream : Void*) : Int32
  fun cogni_rmsnorm_pack16_dev(x : UInt64, norm : UInt64, out : UInt64, w_type : UInt32, image : UInt64, dim : UInt32,
                               tokens : UInt32, eps : Float32, stream : Void*) : Int32
  fun cogni_add_rmsnorm_pack16_dev(x : UInt64, add : UInt64, norm : UInt64, residual_out : UInt64, normed_out : UInt64,
                                   w_type : UInt32, image : UInt64, dim : UInt32, tokens : UInt32, eps : Float32,
                                   stream : Void*) : Int32
  fun cogni_rmsnorm_gemm_pack_dev(x : UInt64, norm : UInt64, out : UInt64, w_type : UInt32, workspace : UInt64,
                                  workspace_bytes : LibC::SizeT, dim : UInt32, tokens : UInt32, eps : Float32, stream : Void*) : Int32
  fun cogni_add_rmsnorm_gemm_pack_dev(x : UInt64, add : UInt64, norm : UInt64, residual_out : UInt64, normed_out : UInt64,
                                      w_type : UInt32, workspace : UInt64, workspace_bytes : LibC::SizeT, dim : UInt32,
                                      tokens : UInt32, eps : Float32, stream : Void*) : Int32
  fun cogni_embed_dev(w_raw : UInt64, w_type : UInt32, token_ids : UInt64, output : UInt64, history : UInt64,
                      token_index : UInt32, hidden_dim : UInt32, vocab_size : UInt32, stream : Void*) : Int32
  fun cogni_gemv_top1_partials(w_type : UInt32, out_dim : UInt32) : UInt32
  fun cogni_gemv_packed_top1_dev(w_raw : UInt64, w_type : UInt32, image : UInt64, partial_ids : UInt64, partial_values : UInt64,
                                 top1_ids : UInt64, top1_values : UInt64, in_dim : UInt32, out_dim : UInt32, tokens : UInt32,
                                 stream : Void*) : Int32
  fun cogni_gemv_top1_dev(w_raw : UInt64, w_type : UInt32, x : UInt64, partial_ids : UInt64, partial_values : UInt64,
                          top1_ids : UInt64, top1_values : UInt64, in_dim : UInt32, out_dim : UInt32, tokens : UInt32,
                          stream : Void*) : Int32
  fun cogni_gemm_workspace_bytes(w_type : UInt32, in_dim : UInt32, tokens : UInt32) : LibC::SizeT
  fun cogni_gemm_workspace_bytes_split(w_type : UInt32, in_dim : UInt32, out_dim : UInt32, tokens : UInt32) : LibC::SizeT
  fun cogni_gemm_dev(w_raw : UInt64, w_type : UInt32, x : UInt64, bias : UInt64, out : UInt64,
                     in_dim : UInt32, out_dim : UInt32, tokens : UInt32,
                     workspace : UInt64, workspace_bytes : LibC::SizeT, stream : Void*) : Int32
  fun cogni_gemm_pack_dev(x : UInt64, w_type : UInt32, in_dim : UInt32, tokens : UInt32,
                          workspace : UInt64, workspace_bytes : LibC::SizeT, stream : Void*) : Int32
  fun cogni_gemm_packed_dev(w_raw : UInt64, w_type : UInt32, workspace : UInt64, workspace_bytes : LibC::SizeT, bias : UInt64,
                            out : UInt64, in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemm_packed_add_dev(w_raw : UInt64, w_type : UInt32, workspace : UInt64, workspace_bytes : LibC::SizeT, residual : UInt64,
                                out : UInt64, in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemm_packed_swiglu_dev(w_gate : UInt64, w_up : UInt64, w_type : UInt32, workspace : UInt64, workspace_bytes : LibC::SizeT,
                                   out : UInt64, in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemv_pack16_dev(x : UInt64, w_type : UInt32, in_dim : UInt32, tokens : UInt32, image : UInt64, stream : Void*) : Int32
  fun cogni_gemv_packed16_dev(w_raw : UInt64*, w_type : UInt32, image : UInt64, residual : UInt64, out : UInt64*, out_dims : UInt32*,
                              count : UInt32, in_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemv_packed16_swiglu_dev(w_gate : UInt64, w_up : UInt64, w_type : UInt32, image : UInt64, out : UInt64, in_dim : UInt32,
                                     out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemm_packed_many_dev(w_raw : UInt64*, w_type : UInt32, workspace : UInt64, workspace_bytes : LibC::SizeT, outs : UInt64*,
                                 out_dims : UInt32*, count : UInt32, in_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemm_packed_swiglu_pack_dev(w_gate : UInt64, w_up : UInt64, w_type : UInt32, workspace : UInt64, workspace_bytes : LibC::SizeT,
                                        out : UInt64, next_type : UInt32, next_workspace : UInt64, next_workspace_bytes : LibC::SizeT,
                                        in_dim : UInt32, out_dim : UInt32, tokens : UInt32, stream : Void*) : Int32
  fun cogni_gemm_plan(w_type : UInt32, in_dim : UInt32, out_dim : UInt32, tokens : UInt32, workspace_bytes : LibC::SizeT,
                      kernel : UInt8**, grid_x : UInt32*, grid_y : UInt32*, block_x : UInt32*) : Int32
  fun cogni_set_gemm_threshold(tokens : Int32) : Int32
  fun cogni_get_gemm_threshold : Int32
  fun cogni_block_bytes(type : UInt32) : Int32
  fun cogni_block_elements(type : UInt32) : Int32
  fun cogni_data_bytes(type : UInt32, n_elements : Int64) : Int64
  fun cogni_quant_shutdown : Int32
  fun cogni_matmul_dev(w_raw : UInt64, w_type : UInt32, x : UInt64, bias : UInt64, out : UInt64,
                       in_dim : UInt32, out_dim : UInt32, tokens : UInt32,
                       workspace : UInt64, workspace_bytes : LibC::SizeT, stream : Void*) : Int32
  fun cogni_dequantize(data : Void*, data_bytes : LibC::SizeT, type : UInt32, n_elements : Int64, out : Float32*) : Int32
  fun cogni_matmul_add(x : Float32*, rows : Int32, in_dim : Int32, w_raw : Void*, w_bytes : LibC::SizeT,
                       w_type : UInt32, out_dim : Int32, bias : Float32*, result : Float32*) : Int32
  fun cogni_weight_create(qw : Void**, raw : Void*, raw_bytes : LibC::SizeT, type : UInt32, out_dim : Int32, in_dim : Int32) : Int32
  fun cogni_weight_device_ptr(qw : Void*) : UInt64
  fun cogni_weight_matmul(qw : Void*, x : Float32*, rows : Int32, bias : Float32*, result : Float32*) : Int32
  fun cogni_weight_matvec_many(qws : Void**, count : Int32, x : Float32*, results : Float32**) : Int32
  fun cogni_weight_destroy(qw : Void*) : Int32
  fun cogni_last_error : UInt8*
end

require "../cuda/driver"   # for the backend-neutral ML::CUDA::ResidentSequenceRunner only

module ML::HIP
  alias DevicePtr = LibCogniHIP::Deviceptr
  @@current_stream = Pointer(Void).null

  def self.check!(code : Int32, what : String) : Nil
    raise "#{what} failed with HIP error #{code}" unless code == 0
  end

  def self.current_stream : Void*
    @@current_stream
  end

  class Context
    getter device_name : String
    getter arch : String
    getter compute_capability_major : Int32
    getter compute_capability_minor : Int32

    def self.create(ordinal : Int32 = 0) : self
      ML::HIP.check! LibCogniHIP.mlhip_init(0_u32), "hipInit"
      device = 0
      ML::HIP.check! LibCogniHIP.mlhip_device_get(pointerof(device), ordinal), "hipDeviceGet"
      buf = Bytes.new(256)
      ML::HIP.check! LibCogniHIP.mlhip_device_get_name(buf.to_unsafe, buf.size, device), "hipDeviceGetName"
      device_name = String.new(buf.to_unsafe).strip
      ML::HIP.check! LibCogniHIP.mlhip_device_get_arch(buf.to_unsafe, buf.size, device), "hipGetDeviceProperties"
      arch = String.new(buf.to_unsafe).strip
      cc_major = 0
      cc_minor = 0
      ML::HIP.check! LibCogniHIP.mlhip_device_compute_capability(pointerof(cc_major), pointerof(cc_minor), device), "hipDeviceComputeCapability"
      handle = Pointer(Void).null
      ML::HIP.check! LibCogniHIP.mlhip_ctx_create(pointerof(handle), 0_u32, device), "hipCtxCreate"
      new(handle, device_name, arch, cc_major, cc_minor)
    end

    def initialize(@handle : Void*, @device_name : String, @arch : String,
                   @compute_capability_major : Int32, @compute_capability_minor : Int32)
      @closed = false
    end

    def close : Nil
      return if @closed
      LibCogniHIP.mlhip_ctx_destroy(@handle) unless @handle.null?
      @closed = true
    end
  end

  class DeviceBuffer
    getter ptr : DevicePtr
    getter bytesize : LibC::SizeT

    def initialize(@bytesize : LibC::SizeT)
      @ptr = 0_u64
      ML::HIP.check! LibCogniHIP.mlhip_mem_alloc(pointerof(@ptr), @bytesize), "hipMalloc"
      @closed = false
    end

    def close : Nil
      return if @closed
      LibCogniHIP.mlhip_mem_free(@ptr) unless @ptr == 0_u64
      @closed = true
    end
  end

  class HIPModule
    # The image is a gfx950 code object (bytes), where CUDAModule.load takes PTX text.
    def self.load(image : Bytes, label : String) : self
      handle = Pointer(Void).null
      ML::HIP.check! LibCogniHIP.mlhip_module_load_data(pointerof(handle), image.to_unsafe.as(Void*)), "hipModuleLoadData(#{label})"
      new(handle)
    end

    # The code object embedded in libcogni_hip.so.
    def self.load_builtin : self
      image = Pointer(Void).null
      size = LibC::SizeT.new(0)
      ML::HIP.check! LibCogniHIP.cogni_quant_code_object(pointerof(image), pointerof(size)), "cogni_quant_code_object"
      load(Bytes.new(image.as(UInt8*), size), "cogni_quant_gfx950")
    end

    def initialize(@handle : Void*)
      @closed = false
    end

    def function(name : String) : KernelFunction
      fn = Pointer(Void).null
      ML::HIP.check! LibCogniHIP.mlhip_module_get_function(pointerof(fn), @handle, name), "hipModuleGetFunction(#{name})"
      KernelFunction.new(fn, name)
    end

    def close : Nil
      return if @closed
      LibCogniHIP.mlhip_module_unload(@handle) unless @handle.null?
      @closed = true
    end
  end

  class KernelFunction
    getter handle : Void*
    getter name : String

    def initialize(@handle : Void*, @name : String)
    end

    def attribute(attr : FunctionAttribute) : Int32
      value = 0
      ML::HIP.check! LibCogniHIP.mlhip_func_get_attribute(pointerof(value), attr.value, @handle),
        "hipFuncGetAttribute(#{@name}, #{attr})"
      value
    end
  end

  enum FunctionAttribute
    MaxThreadsPerBlock            = 0
    SharedSizeBytes               = 1
    ConstSizeBytes                = 2
    LocalSizeBytes                = 3
    NumRegs                       = 4
    PtxVersion                    = 5
    BinaryVersion                 = 6
    CacheModeCa                   = 7
    MaxDynamicSharedSizeBytes     = 8
    PreferredSharedMemoryCarveout = 9
  end

  class HIPStream
    getter handle : Void*

    def initialize(flags : UInt32 = 0_u32)
      @handle = Pointer(Void).null
      ML::HIP.check! LibCogniHIP.mlhip_stream_create(pointerof(@handle), flags), "hipStreamCreate"
      @closed = false
    end

    def synchronize : Nil
      ML::HIP.check! LibCogniHIP.mlhip_stream_synchronize(@handle), "hipStreamSynchronize"
    end

    def begin_capture(mode : Int32 = 1) : Nil
      ML::HIP.check! LibCogniHIP.mlhip_stream_begin_capture(@handle, mode), "hipStreamBeginCapture"
    end

    def end_capture : HIPGraph
      graph = Pointer(Void).null
      ML::HIP.check! LibCogniHIP.mlhip_stream_end_capture(@handle, pointerof(graph)), "hipStreamEndCapture"
      HIPGraph.new(graph)
    end

    def close : Nil
      return if @closed
      LibCogniHIP.cogni_gemv_release_stream(@handle) unless @handle.null?   # the activation image kept for this stream
      LibCogniHIP.mlhip_stream_destroy(@handle) unless @handle.null?
      @closed = true
    end
  end

  class HIPGraph
    def initialize(@handle : Void*)
      @closed = false
    end

    def instantiate : HIPGraphExec
      exec = Pointer(Void).null
      ML::HIP.check! LibCogniHIP.mlhip_graph_instantiate(pointerof(exec), @handle, 0_u64), "hipGraphInstantiateWithFlags"
      HIPGraphExec.new(exec)
    end

    def close : Nil
      return if @closed
      LibCogniHIP.mlhip_graph_destroy(@handle) unless @handle.null?
      @closed = true
    end
  end

  class HIPGraphExec
    def initialize(@handle : Void*)
      @closed = false
    end

    def launch(stream : HIPStream) : Nil
      ML::HIP.check! LibCogniHIP.mlhip_graph_launch(@handle, stream.handle), "hipGraphLaunch"
    end

    def upload(stream : HIPStream) : Nil
      ML::HIP.check! LibCogniHIP.mlhip_graph_upload(@handle, stream.handle), "hipGraphUpload"
    end

    def close : Nil
      return if @closed
      LibCogniHIP.mlhip_graph_exec_destroy(@handle) unless @handle.null?
      @closed = true
    end
  end

  def self.with_stream(stream : HIPStream) : Nil
    previous = @@current_stream
    @@current_stream = stream.handle
    begin
      yield
    ensure
      @@current_stream = previous
    end
  end

  def self.copy_htod!(dst : DevicePtr, src : Void*, bytesize : LibC::SizeT, what : String) : Nil
    check! LibCogniHIP.mlhip_memcpy_htod(dst, src, bytesize), "hipMemcpyHtoD(#{what})"
  end

  def self.copy_dtoh!(dst : Void*, src : DevicePtr, bytesize : LibC::SizeT, what : String) : Nil
    check! LibCogniHIP.mlhip_memcpy_dtoh(dst, src, bytesize), "hipMemcpyDtoH(#{what})"
  end

  def self.copy_dtod!(dst : DevicePtr, src : DevicePtr, bytesize : LibC::SizeT, what : String) : Nil
    check! LibCogniHIP.mlhip_memcpy_dtod(dst, src, bytesize), "hipMemcpyDtoD(#{what})"
  end

  def self.synchronize!(what : String = "hipDeviceSynchronize") : Nil
    check! LibCogniHIP.mlhip_ctx_synchronize, what
  end

  def self.launch!(fn : KernelFunction,
                   grid_x : UInt32, grid_y : UInt32, grid_z : UInt32,
                   block_x : UInt32, block_y : UInt32, block_z : UInt32,
                   params : Void**, label : String,
                   shared_mem_bytes : UInt32 = 0_u32) : Nil
    check! LibCogniHIP.mlhip_launch_kernel(fn.handle, grid_x, grid_y, grid_z,
      block_x, block_y, block_z, shared_mem_bytes, @@current_stream,
      params, Pointer(Void*).null), "hipModuleLaunchKernel(#{label})"
  end

  # The resident-sequence facade is backend neutral in the reference (src/ml/cuda/driver.cr:288-342: five procs and a
  # token count, no driver call), so the HIP runners use that very class rather than a second copy of it. Requiring
  # the CUDA binding file does not link libcuda: Crystal only links a `lib` whose funs are called.
  alias ResidentSequenceRunner = ML::CUDA::ResidentSequenceRunner

  # The GPU arm of the projection router: same shape as Qwen35Metal.matmul(qw, x, batch) : Array(Float32)?
  # (src/ml/gguf/qwen35_cpu.cr:1398-1412, 1478-1490). nil = not eligible, fall back to QuantMatmul.matmul_add.
  module QuantMatmulHIP
    def self.matmul(raw : Bytes, type_id : UInt32, out_dim : Int32, in_dim : Int32,
                    x : Array(Float32), batch : Int32, bias : Array(Float32)? = nil) : Array(Float32)?
      return nil unless {8_u32, 12_u32, 13_u32, 14_u32}.includes?(type_id)
      return nil unless out_dim >= 256 && in_dim >= 256
      result = Array(Float32).new(batch * out_dim, 0.0_f32)
      code = LibCogniHIP.cogni_matmul_add(x.to_unsafe, batch, in_dim, raw.to_unsafe.as(Void*), raw.size,
        type_id, out_dim, bias ? bias.to_unsafe : Pointer(Float32).null, result.to_unsafe)
      raise String.new(LibCogniHIP.cogni_last_error) unless code == 0
      result
    end
  end
end
