classdef Conv2DLayer < Conv2DLayer
    % Conv2DLayer whose ImageStar reach (Conv2DLayer.m:559-601, 862-886) runs on the device.
    properties (Transient)
        devW = uint64(0);   % nnvhip_conv2d* handle
    end
    methods
        function obj = Conv2DLayer(varargin)
            obj = obj@Conv2DLayer(varargin{:});
        end
        function S = reach_star_multipleInputs(obj, inputs, option) %#ok<INUSD>
            if obj.devW == 0
                obj.devW = nnvhip_mex('conv2d_create', double(obj.Weights), double(obj.Bias(:)), ...
                    double(obj.PaddingSize), double(obj.Stride), double(obj.DilationFactor));
            end
            n = length(inputs);
            hs = zeros(1, n, 'uint64');
            for i = 1:n
                if ~isa(inputs(i), 'ImageStar')
                    error('The input is not an ImageStar object');
                end
                if inputs(i).numChannel ~= obj.NumChannels
                    error("Input set contains %d channels while the convolutional layers has %d channels", inputs(i).numChannel, obj.NumChannels);
                end
                hs(i) = inputs(i).dev.h;
            end
            H = inputs(1).height; W = inputs(1).width;
            out = nnvhip_mex('affine_conv2d', obj.devW, H, W, hs);
            p = obj.PaddingSize; f = obj.FilterSize; s = obj.Stride; dl = obj.DilationFactor;
            ho = floor((H + p(1) + p(2) - (f(1)-1)*dl(1) - 1)/s(1) + 1);   % Conv2DLayer.m:1134-1135
            wo = floor((W + p(3) + p(4) - (f(2)-1)*dl(2) - 1)/s(2) + 1);
            for i = n:-1:1
                S(i) = nnvhip.ImageStar(nnvhip.DeviceSet(out(i)), ho, wo, obj.NumFilters);
            end
        end
        function S = reach_star_single_input(obj, input)
            S = obj.reach_star_multipleInputs(input, 'single');
        end
        function delete(obj)
            if obj.devW ~= 0, nnvhip_mex('conv2d_destroy', obj.devW); end
        end
    end
end
