import torch


class Bias(torch.nn.Module):
    """Learned per-feature offset, parameter ``bias_`` [1, F] (pccnn_lib/pc/layers/Bias.py:3-29)."""

    def __init__(self, p_num_features):
        super(Bias, self).__init__()
        self.bias_ = torch.nn.Parameter(torch.zeros(1, p_num_features))

    def forward(self, p_in_features):
        return p_in_features + self.bias_


class GroupNormalization(torch.nn.Module):
    """Per-cloud group normalisation of point features, parameters ``gamma_`` and ``betas_`` [1, F]
    (pccnn_lib/pc/layers/GroupNormalization.py:5-60).  The reference views the [N, F] features as rows of
    ``groups`` values (feature f = chunk * groups + column) and normalises every column with the mean and variance
    over all rows of the point's cloud; here that is a [N, F / groups, groups] view whose statistics are taken over
    the points of a cloud and the chunks, which is the same set of values per column."""

    def __init__(self, p_num_features, p_num_groups):
        super(GroupNormalization, self).__init__()
        self.num_features_, self.num_groups_ = p_num_features, p_num_groups
        self.gamma_ = torch.nn.Parameter(torch.ones(1, p_num_features))
        self.betas_ = torch.nn.Parameter(torch.zeros(1, p_num_features))

    def forward(self, p_feats, p_pc):
        columns = self.num_groups_
        chunks = self.num_features_ // columns
        cloud_of = p_pc.batch_ids_.to(torch.int64)
        clouds = p_pc.batch_size_host()
        values = p_feats.reshape(-1, chunks, columns)
        weight = torch.bincount(cloud_of, minlength=clouds).clamp(min=1).to(values.dtype).reshape(-1, 1) * chunks

        def cloud_mean(p_values):
            total = torch.zeros((clouds, columns), dtype=values.dtype, device=values.device)
            return total.index_add(0, cloud_of, p_values.sum(dim=1)) / weight

        centred = values - cloud_mean(values)[cloud_of].unsqueeze(1)
        spread = cloud_mean(centred * centred)[cloud_of].unsqueeze(1)
        normed = centred / torch.sqrt(spread + 1e-8)
        return normed.reshape(-1, self.num_features_) * self.gamma_ + self.betas_
