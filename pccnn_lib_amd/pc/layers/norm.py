import torch


class Bias(torch.nn.Module):
    """Learned per-feature offset, parameter ``bias_`` [1, F] (pccnn_lib/pc/layers/Bias.py:3-29)."""

    def __init__(self, p_num_features):
        super(Bias, self).__init__()
        self.bias_ = torch.nn.Parameter(torch.zeros(1, p_num_features))

    def forward(self, p_in_features):
        return p_in_features + self.bias_


def _mean_per_batch(p_values, p_ids, p_num_batches):
    sums = torch.zeros((p_num_batches, p_values.shape[1]), dtype=p_values.dtype, device=p_values.device)
    sums = sums.index_add(0, p_ids, p_values)
    counts = torch.bincount(p_ids, minlength=p_num_batches).clamp(min=1).to(p_values.dtype)
    return sums / counts.reshape(-1, 1)


class GroupNormalization(torch.nn.Module):
    """Per-cloud group normalisation of point features, parameters ``gamma_`` and ``betas_`` [1, F].  As in the
    reference the [N, F] features are viewed as [N * F / groups, groups] rows before the per-cloud statistics
    are taken (pccnn_lib/pc/layers/GroupNormalization.py:5-60)."""

    def __init__(self, p_num_features, p_num_groups):
        super(GroupNormalization, self).__init__()
        self.num_features_ = p_num_features
        self.num_groups_ = p_num_groups
        self.gamma_ = torch.nn.Parameter(torch.ones(1, p_num_features))
        self.betas_ = torch.nn.Parameter(torch.zeros(1, p_num_features))

    def forward(self, p_feats, p_pc):
        eps_val = 1e-8
        group_size = self.num_features_ // self.num_groups_
        cur_feats = p_feats.reshape((-1, self.num_groups_))
        ids = p_pc.batch_ids_.reshape((-1, 1)).repeat(1, group_size).to(torch.int64).reshape((-1,))
        num_batches = p_pc.batch_size_host()
        means = _mean_per_batch(cur_feats, ids, num_batches)[ids]
        variances = _mean_per_batch((cur_feats - means) ** 2, ids, num_batches)[ids]
        cur_feats = (cur_feats - means) / torch.sqrt(variances + eps_val)
        return cur_feats.reshape((-1, self.num_features_)) * self.gamma_ + self.betas_
