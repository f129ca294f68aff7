function net = prepare(net)
% NNVHIP.PREPARE  Swap the hot-path layers of an NN for their device-backed subclasses.
%   net = nnvhip.prepare(net) replaces every FullyConnectedLayer / Conv2DLayer / ReluLayer /
%   BatchNormalizationLayer / AveragePooling2DLayer / FlattenLayer / ImageInputLayer in net.Layers
%   by its nnvhip.* subclass - the same
%   per-layer replacement NNV itself performs in NN.params2gpu -> layer.toGPU (NN.m:1257-1263).
%   NN.reach, reachOptions and the layers' reach signatures are untouched.  Typical use:
%
%       net = nnvhip.prepare(net);
%       I   = nnvhip.ImageStar(lb_image, ub_image);          % or nnvhip.Star(lb, ub)
%       R   = net.reach(I, struct('reachMethod','relax-star-area','relaxFactor',1));
%       [lb, ub] = R.estimateRanges;                         % LP-free output bounds
%       S   = R.gather();                                    % dense NNV set (V, C, d) on the host
for i = 1:numel(net.Layers)
    L = net.Layers{i};
    if isa(L, 'FullyConnectedLayer') && ~isa(L, 'nnvhip.FullyConnectedLayer')
        net.Layers{i} = nnvhip.FullyConnectedLayer(L.Name, L.Weights, L.Bias);
    elseif isa(L, 'Conv2DLayer') && ~isa(L, 'nnvhip.Conv2DLayer')
        net.Layers{i} = nnvhip.Conv2DLayer(L.Name, L.Weights, L.Bias, L.PaddingSize, L.Stride, L.DilationFactor);
    elseif isa(L, 'ReluLayer') && ~isa(L, 'nnvhip.ReluLayer')
        net.Layers{i} = nnvhip.ReluLayer(L.Name, L.NumInputs, L.InputNames, L.NumOutputs, L.OutputNames);
    elseif isa(L, 'BatchNormalizationLayer') && ~isa(L, 'nnvhip.BatchNormalizationLayer')
        net.Layers{i} = nnvhip.BatchNormalizationLayer('Name', L.Name, 'NumChannels', L.NumChannels, ...
            'TrainedMean', L.TrainedMean, 'TrainedVariance', L.TrainedVariance, 'Epsilon', L.Epsilon, ...
            'Offset', L.Offset, 'Scale', L.Scale);
    elseif isa(L, 'AveragePooling2DLayer') && ~isa(L, 'nnvhip.AveragePooling2DLayer')
        net.Layers{i} = nnvhip.AveragePooling2DLayer(L.Name, L.PoolSize, L.Stride, L.PaddingSize);
    elseif isa(L, 'FlattenLayer') && ~isa(L, 'nnvhip.FlattenLayer')
        F = nnvhip.FlattenLayer(L.Name); F.Type = L.Type;
        net.Layers{i} = F;
    elseif isa(L, 'ImageInputLayer') && ~isa(L, 'nnvhip.ImageInputLayer')
        net.Layers{i} = nnvhip.ImageInputLayer(L.Name, L.InputSize, L.Normalization, L.NormalizationDimension, ...
            L.Mean, L.StandardDeviation, L.Min, L.Max);
    end
end
end
