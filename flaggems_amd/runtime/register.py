"""Registration of Python kernels over ATen operators
(behaviour of src/flag_gems/runtime/register.py:5-61 and runtime/error.py:12-15)."""


class Register:
    def __init__(self, config, user_unused_ops_list=None, cpp_patched_ops_list=None, lib=None):
        from . import device, get_device_unused_op

        self.device = device
        self.lib = lib
        self.reg_key = device.dispatch_key
        self.all_ops = []
        self.vendor_unused_ops_list = get_device_unused_op()
        self.unused_ops = list(user_unused_ops_list or []) + self.vendor_unused_ops_list
        self.cpp_patched_ops_list = set(cpp_patched_ops_list or [])
        self.config = config
        self.config_filter()
        self.for_each()

    def config_filter(self):
        # rows are filtered by the *python function name*, as in the reference
        self.config = [
            (key, fn)
            for key, fn in self.config
            if fn.__name__ not in self.unused_ops and key not in self.cpp_patched_ops_list
        ]

    def register_impl(self, key, fn):
        self.all_ops.append(key)
        self.lib.impl(key, fn, self.reg_key)

    def for_each(self):
        try:
            for key, fn in self.config:
                self.register_impl(key, fn)
        except Exception as e:
            raise RuntimeError(e, "An error was encountered while registering the triton operator.")

    def get_all_ops(self):
        return self.all_ops

    def get_unused_ops(self):
        return self.unused_ops

    def get_vendor_name(self):
        return self.device.vendor_name

    def get_current_device(self):
        return self.device.name
