"""Drop-in for the reference's `codegen_tensops_cuda` extension
(extensions/codegen_tensops/codegen_tensops.cpp:1980-2011).  The Bee and Cow
families and the Ant16 forward functions run on the HIP kernels; the Ant16 backward functions
(training of the legacy architectures) raise NotImplementedError."""
import importlib

_ops = importlib.import_module("learned-dynamics_amd.ops")

bee_fwd_cuda = _ops.bee_fwd
bee_bwl_cuda = _ops.bee_bwl
bee_bwr_cuda = _ops.bee_bwr
cow_o0_fwd_cuda = _ops.cow_o0_fwd
cow_o0_bwl_cuda = _ops.cow_o0_bwl
cow_o0_bwr_cuda = _ops.cow_o0_bwr
cow_o1_fwd_cuda = _ops.cow_o1_fwd
cow_o1_bwl_cuda = _ops.cow_o1_bwl
cow_o1_bwr_cuda = _ops.cow_o1_bwr


def set_kern_attributes():
    """The reference raises the dynamic shared-memory limit for Ant16 here; nothing to do."""
    return None


def _ant16_unavailable(name):
    def fn(*args, **kwargs):
        raise NotImplementedError(f"{name}: only the forward functions of the Ant16 family are implemented")
    fn.__name__ = name
    return fn


ant16_o0_cuda = _ops.ant16_o0
ant16_o1_cuda = _ops.ant16_o1
ant16_o2_cuda = _ops.ant16_o2
ant16_oc_cuda = _ops.ant16_oc

for _o in ("o0", "o1", "o2", "oc"):
    for _suffix in ("_backward", "_backleft", "_wtsback"):
        _name = f"ant16_{_o}{_suffix}_cuda"
        globals()[_name] = _ant16_unavailable(_name)
for _suffix in ("", "_backward", "_backleft", "_wtsback"):
    _name = f"fused_tensor_prods_example{_suffix}_cuda"
    globals()[_name] = _ant16_unavailable(_name)
