classdef FlattenLayer < FlattenLayer
    % FlattenLayer on device-resident ImageStars (FlattenLayer.m:118-170, 178-243): the MATLAB-style
    % flatten is a reshape of the same device buffer; the Keras / ONNX C-style variants are a row
    % permutation.
    methods
        function obj = FlattenLayer(varargin)
            obj = obj@FlattenLayer(varargin{:});
        end
        function S = reach_multipleInputs(obj, inputs, option) %#ok<INUSD>
            if isa(inputs(1), 'Star')
                S = inputs;      % already flat
                return;
            end
            n = length(inputs);
            h = inputs(1).height; w = inputs(1).width; c = inputs(1).numChannel; N = h*w*c;
            if strcmp(obj.Type, 'nnet.cnn.layer.FlattenLayer')
                for i = n:-1:1, S(i) = nnvhip.ImageStar(inputs(i).dev, 1, 1, N); end
                return;
            end
            src = reshape(obj.evaluate(reshape(1:N, h, w, c)), [], 1);   % where every flattened row comes from
            hs = zeros(1, n, 'uint64');
            for i = 1:n, hs(i) = inputs(i).dev.h; end
            out = nnvhip_mex('permute_rows', double(src), hs);
            for i = n:-1:1, S(i) = nnvhip.ImageStar(nnvhip.DeviceSet(out(i)), 1, 1, N); end
        end
        function S = reach_single_input(obj, in_set)
            S = obj.reach_multipleInputs(in_set, 'single');
        end
    end
end
