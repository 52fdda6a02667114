"""`Registry.build({'type', 'kwargs'})` convention of the reference
(llm/utils/general/registry.py:19-121, registry_factory.py:1-28), reduced to the two registries the
decoder-layer step uses."""


class Registry(dict):
    def register(self, module_name=None, module=None):
        if module is not None:
            assert module_name is not None
            self._register(module_name, module)
            return None

        def register_fn(fn):
            self._register(fn.__name__ if module_name is None else module_name, fn)
            return fn

        return register_fn

    def _register(self, name, module):
        assert name not in self, name
        self[name] = module

    def get(self, module_name):
        assert module_name in self, "{} is not supported, avaiables are:{}".format(module_name, list(self))
        return self[module_name]

    def build(self, cfg):
        obj_type = cfg["type"]
        obj_kwargs = cfg.get("kwargs", {})
        assert obj_type in self, "{} is not supported, avaiables are:{}".format(obj_type, list(self))
        return self[obj_type](**obj_kwargs)

    def query(self):
        return self.keys()


MODULE_ZOO_REGISTRY = Registry()
LOSS_REGISTRY = Registry()
