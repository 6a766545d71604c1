"""Drop-in for the reference's `codegen_tensops_cuda` extension
(extensions/codegen_tensops/codegen_tensops.cpp:1980-2011): the Bee, Cow and Ant16
families, forward and backward, on the HIP kernels."""
import importlib

_ops = importlib.import_module("learned-dynamics_amd.ops")
_a16 = importlib.import_module("learned-dynamics_amd.ant16_backward")

# Bee and Cow: the package's PyTorch C++ binding (csrc/torch_binding.cpp)
_ext = importlib.import_module("learned-dynamics_amd._lib").load_torch_ext()
bee_fwd_cuda = _ext.bee_fwd_cuda
bee_bwl_cuda = _ext.bee_bwl_cuda
bee_bwr_cuda = _ext.bee_bwr_cuda
cow_o0_fwd_cuda = _ext.cow_o0_fwd_cuda
cow_o0_bwl_cuda = _ext.cow_o0_bwl_cuda
cow_o0_bwr_cuda = _ext.cow_o0_bwr_cuda
cow_o1_fwd_cuda = _ext.cow_o1_fwd_cuda
cow_o1_bwl_cuda = _ext.cow_o1_bwl_cuda
cow_o1_bwr_cuda = _ext.cow_o1_bwr_cuda


def set_kern_attributes():
    """The reference raises the dynamic shared-memory limit for Ant16 here; nothing to do."""
    return None


ant16_o0_cuda = _ops.ant16_o0
ant16_o1_cuda = _ops.ant16_o1
ant16_o2_cuda = _ops.ant16_o2
ant16_oc_cuda = _ops.ant16_oc


def _checked(name, fn):
    def wrapper(*tensors):
        for k, t in enumerate(tensors):
            _ops._check_input(t, f"{name} argument {k}")
        return fn(*tensors)
    wrapper.__name__ = name
    return wrapper


for _o in ("o0", "o1", "o2"):
    for _suffix, _fn in (("_backward", _a16.backward), ("_backleft", _a16.backleft), ("_wtsback", _a16.wtsback)):
        _name = f"ant16_{_o}{_suffix}_cuda"
        globals()[_name] = _checked(_name, (lambda f, o: lambda *a: f(o, *a))(_fn, _o))
ant16_oc_backward_cuda = _checked("ant16_oc_backward_cuda", _a16.oc_backward)
ant16_oc_backleft_cuda = _checked("ant16_oc_backleft_cuda", _a16.oc_backleft)
ant16_oc_wtsback_cuda = _checked("ant16_oc_wtsback_cuda", _a16.oc_wtsback)
# the generated example with nine product types of mixed output rank (codegen_tensops.cpp:1981-1984)
fused_tensor_prods_example_cuda = _checked("fused_tensor_prods_example_cuda", _a16.example_forward)
fused_tensor_prods_example_backward_cuda = _checked("fused_tensor_prods_example_backward_cuda", _a16.example_backward)
fused_tensor_prods_example_backleft_cuda = _checked("fused_tensor_prods_example_backleft_cuda", _a16.example_backleft)
fused_tensor_prods_example_wtsback_cuda = _checked("fused_tensor_prods_example_wtsback_cuda", _a16.example_wtsback)
