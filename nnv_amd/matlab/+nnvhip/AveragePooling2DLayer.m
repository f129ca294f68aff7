classdef AveragePooling2DLayer < AveragePooling2DLayer
    % AveragePooling2DLayer whose ImageStar reach (AveragePooling2DLayer.m:424-463) runs on the
    % device: vl_nnpool's mean over the part of each window that lies inside the image.
    properties (Transient)
        devL = uint64(0);
    end
    methods
        function obj = AveragePooling2DLayer(varargin)
            obj = obj@AveragePooling2DLayer(varargin{:});
        end
        function S = reach_star_multipleInputs(obj, inputs, option) %#ok<INUSD>
            if obj.devL == 0
                obj.devL = nnvhip_mex('avgpool2d_create', double(obj.PoolSize), double(obj.Stride), double(obj.PaddingSize));
            end
            n = length(inputs);
            hs = zeros(1, n, 'uint64');
            for i = 1:n
                if ~isa(inputs(i), 'ImageStar'), error('The input is not an ImageStar object'); end
                hs(i) = inputs(i).dev.h;
            end
            [out, ho, wo] = nnvhip_mex('affine_avgpool2d', obj.devL, inputs(1).height, inputs(1).width, hs);
            for i = n:-1:1
                S(i) = nnvhip.ImageStar(nnvhip.DeviceSet(out(i)), ho, wo, inputs(i).numChannel);
            end
        end
        function S = reach_star_single_input(obj, input)
            S = obj.reach_star_multipleInputs(input, 'single');
        end
        function delete(obj)
            if obj.devL ~= 0, nnvhip_mex('avgpool2d_destroy', obj.devL); end
        end
    end
end
