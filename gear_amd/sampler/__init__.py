from .global_sampler import TopKSampler, UniformSampler, WeightedSampler

# OfflineLoader documents sampling_method "Topk" (gear/loader/offline_loader.py:44,61) and looks
# up "<method>Sampler" (:102-104); the class is TopKSampler, so that spelling needs this alias.
TopkSampler = TopKSampler

__all__ = ["UniformSampler", "WeightedSampler", "TopKSampler", "TopkSampler"]
