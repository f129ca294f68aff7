function result = nnv_cpu_reach(fixture_mat, method, threads)
% NNV_CPU_REACH  Time NNV's own CPU reach on one of the benchmark configurations.
%   result = nnv_cpu_reach('cfg2.mat', 'relax-star-area', 8)
%   fixture_mat is written by  python -m nnv_amd.export_fixture <k> <file.mat>  and holds
%   layers (cell of structs: type, W, b, padding, stride, dilation), lb, ub and image_shape.
%   Runs wherever MATLAB + NNV are installed; prints the thread count, per-layer reachTime
%   (NN.m:1542-1545) and total wall-time, and returns the output set for parity checks.
if nargin < 2, method = 'relax-star-area'; end
if nargin >= 3, maxNumCompThreads(threads); end
f = load(fixture_mat);
Ls = cell(1, numel(f.layers));
for i = 1:numel(f.layers)
    L = f.layers{i};
    switch char(L.type)
        case 'fc',   Ls{i} = FullyConnectedLayer(L.W, L.b(:));
        case 'conv', Ls{i} = Conv2DLayer(L.W, reshape(L.b, 1, 1, []), double(L.padding(:)'), double(L.stride(:)'), double(L.dilation(:)'));
        case 'relu', Ls{i} = ReluLayer();
    end
end
net = NN(Ls);
if isfield(f, 'image_shape') && ~isempty(f.image_shape)
    sh = double(f.image_shape(:)');
    I = ImageStar(reshape(f.lb, sh), reshape(f.ub, sh));
else
    I = Star(f.lb(:), f.ub(:));
end
opts = struct('reachMethod', method, 'relaxFactor', 1);
fprintf('maxNumCompThreads = %d\n', maxNumCompThreads);
t = tic; R = net.reach(I, opts); total = toc(t);
fprintf('reach wall-time %.6f s; per layer: %s\n', total, mat2str(net.reachTime, 4));
if isa(R, 'ImageStar'), S = R.toStar; else, S = R; end
[lb, ub] = S.estimateRanges;
result = struct('V', S.V, 'C', S.C, 'd', S.d, 'predicate_lb', S.predicate_lb, 'predicate_ub', S.predicate_ub, ...
    'out_lb', lb, 'out_ub', ub, 'reachTime', net.reachTime, 'total', total, 'threads', maxNumCompThreads);
end
