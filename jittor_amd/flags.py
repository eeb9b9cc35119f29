"""Run-time flags: `jt.flags.<name>` / `jt.flags["<name>"]` and `jt.flag_scope`
(python/jittor/__init__.py flag_scope; the flags themselves are DEFINE_FLAGs of
the reference's core, here only the ones the meta-operator path reads).

amp_reg and auto_mixed_precision_level (alias amp_level) are the
mixed-precision control of python/jittor/src/var.cc:28,65-71; the register
itself lives in dtypes.amp_reg where the inference rules read it.
"""
import contextlib

from . import dtypes


class Flags(dict):
    _AMP_LEVEL = ("auto_mixed_precision_level", "amp_level")

    def __getattr__(self, name):
        if name == "amp_reg":
            return dtypes.amp_reg
        try:
            return self[name]
        except KeyError:
            raise AttributeError("unknown flag %r" % name)

    def __setattr__(self, name, value):
        self[name] = value

    def __getitem__(self, name):
        if name == "amp_reg":
            return dtypes.amp_reg
        if name in self._AMP_LEVEL:
            return dict.get(self, "auto_mixed_precision_level", 0)
        return dict.__getitem__(self, name)

    def __setitem__(self, name, value):
        if name == "amp_reg":
            dtypes.amp_reg = int(value)
        elif name in self._AMP_LEVEL:
            dict.__setitem__(self, "auto_mixed_precision_level", int(value))
            dtypes.amp_reg = dtypes.amp_reg_of_level(int(value))
        elif name not in self:
            raise KeyError("unknown flag %r" % name)
        else:
            dict.__setitem__(self, name, value)


flags = Flags()
for _name, _value in (("enable_conv_match", True), ("enable_reduce_fusion", True), ("enable_broadcast_sink", True),
                      ("enable_matmul_match", True), ("enable_conv_wgrad_kernel", True), ("enable_gather_reduce", True), ("enable_scatter_fusion", True), ("reshape_shares_memory", True), ("enable_replay", True), ("auto_mixed_precision_level", 0),
                      # default compile options of new vars (python/jittor/src/var.cc:19,75): a dict name -> int
                      ("compile_options", {})):
    dict.__setitem__(flags, _name, _value)


@contextlib.contextmanager
def flag_scope(**kw):
    """with jt.flag_scope(amp_reg=2 + 16): ...  -- sets the flags and restores them on exit."""
    saved = {k: flags[k] for k in kw}
    saved_amp = dtypes.amp_reg
    try:
        for k, v in kw.items():
            flags[k] = v
        yield
    finally:
        for k, v in saved.items():
            if k not in Flags._AMP_LEVEL and k != "amp_reg":
                flags[k] = v
            elif k in Flags._AMP_LEVEL:
                dict.__setitem__(flags, "auto_mixed_precision_level", v)
        dtypes.amp_reg = saved_amp
