"""The plug-in registry (reference: src/compressed_tensors/registry/registry.py,
tests/test_registry.py)."""
import pytest

from compressed_tensors_amd import (BaseCompressor, BitmaskCompressor, BitmaskConfig, CompressionFormat,
                                    DenseCompressor, DenseSparsityConfig, Sparse24BitMaskConfig,
                                    SparsityCompressionConfig)
from compressed_tensors_amd.registry import (RegistryMixin, get_from_registry, register, registered_aliases,
                                             registered_names, standardize_lookup_name)


@pytest.mark.parametrize("name,kind", [(CompressionFormat.sparse_bitmask.value, BitmaskConfig),
                                       (CompressionFormat.dense.value, DenseSparsityConfig),
                                       (CompressionFormat.sparse_24_bitmask.value, Sparse24BitMaskConfig)])
def test_configs(name, kind):
    """tests/test_registry.py:27-38"""
    config = SparsityCompressionConfig.load_from_registry(name)
    assert isinstance(config, kind) and config.format == name
    # the fields of a config.json entry, unknown keys aside
    config = SparsityCompressionConfig.load_from_registry(
        name, format=name, targets=["Linear"], global_sparsity=0.5, registry_requires_subclass=False)
    assert isinstance(config, kind) and config.targets == ["Linear"] and config.global_sparsity == 0.5
    with pytest.raises(KeyError, match="Unable to find"):
        SparsityCompressionConfig.load_from_registry("no-such-format")


@pytest.mark.parametrize("name,kind", [(CompressionFormat.sparse_bitmask.value, BitmaskCompressor),
                                       (CompressionFormat.dense.value, DenseCompressor)])
def test_compressors(name, kind):
    """tests/test_registry.py:41-55"""
    compressor = BaseCompressor.load_from_registry(name, config=SparsityCompressionConfig(format="none"))
    assert isinstance(compressor, kind)
    assert isinstance(compressor.config, SparsityCompressionConfig) and compressor.config.format == "none"


def test_names_aliases_and_a_table_per_class():
    class Dataset(RegistryMixin):
        pass

    class Other(RegistryMixin):
        pass

    @Dataset.register()
    class ImageNet_Set(Dataset):
        pass

    @Dataset.register(name="cifar dataset", alias=["cifar-10", "Cifar_100"])
    class Cifar(Dataset):
        pass

    assert standardize_lookup_name("Foo_bar baz") == "foo-bar-baz"
    assert Dataset.registered_names() == ["imagenet-set", "cifar-dataset"]
    assert sorted(Dataset.registered_aliases()) == ["cifar-10", "cifar-100"]
    for name in ("cifar_dataset", "CIFAR DATASET", "cifar-10", "cifar 100"):
        assert Dataset.get_value_from_registry(name) is Cifar
    assert isinstance(Dataset.load_from_registry("ImageNet_Set"), ImageNet_Set)
    assert Cifar.get_value_from_registry("imagenet-set") is ImageNet_Set  # found through the base
    assert Other.registered_names() == []
    with pytest.raises(KeyError):
        Other.get_value_from_registry("cifar-dataset")
    # the same value under its name again: nothing happens; another value: an error
    Dataset.register_value(Cifar, name="cifar-dataset")
    with pytest.raises(RuntimeError, match="already been registered"):
        Dataset.register_value(ImageNet_Set, name="cifar_dataset")
    with pytest.raises(KeyError, match="already been registered"):
        Dataset.register_value(ImageNet_Set, name="third", alias="cifar-10")
    with pytest.raises(KeyError, match="identical to the standardized name"):
        Dataset.register_value(ImageNet_Set, name="fourth", alias="fourth")
    # the functions behind the methods
    register(Other, int, name="an int")
    assert get_from_registry(Other, "an_int") is int and registered_names(Other) == ["an-int"]
    assert registered_aliases(Other) == []


def test_subclass_requirement_and_values_from_files(tmp_path):
    class Strict(RegistryMixin):
        registry_requires_subclass = True

    class Loose(RegistryMixin):
        pass

    with pytest.raises(ValueError, match="not a subclass"):
        Strict.register_value(int, name="int")
    Loose.register_value(int, name="int")
    assert Loose.get_value_from_registry("int") is int

    plugin = tmp_path / "plugin.py"
    plugin.write_text("class Mine:\n    def __init__(self, k=1):\n        self.k = k\nempty = None\n")
    made = Loose.load_from_registry(f"{plugin}:Mine", k=5)
    assert type(made).__name__ == "Mine" and made.k == 5
    with pytest.raises(RuntimeError, match="Unable to find attribute"):
        Loose.get_value_from_registry(f"{plugin}:empty")
    with pytest.raises(ValueError, match="not a subclass"):
        Strict.get_value_from_registry(f"{plugin}:Mine")
