classdef FullyConnectedLayer < FullyConnectedLayer
    % FullyConnectedLayer whose star reach runs on the device.  reach()'s signature and method
    % routing are inherited unchanged (FullyConnectedLayer.m:162-220); only the per-set work
    % (:295-316, 476-512) is replaced, and an array of sets is one batched device call.
    properties (Transient)
        devW = uint64(0);   % nnvhip_fc* handle, created on first use
    end
    methods
        function obj = FullyConnectedLayer(varargin)
            obj = obj@FullyConnectedLayer(varargin{:});
        end
        function S = reach_star_multipleInputs(obj, inputs, option) %#ok<INUSD>
            if obj.devW == 0
                obj.devW = nnvhip_mex('fc_create', double(obj.Weights), double(obj.Bias));
            end
            n = length(inputs);
            hs = zeros(1, n, 'uint64');
            for i = 1:n
                if isa(inputs(i), 'ImageStar')
                    if inputs(i).height*inputs(i).width*inputs(i).numChannel ~= obj.InputSize
                        error('Inconsistency between the size of the input image and the InputSize of the network');
                    end
                elseif ~isa(inputs(i), 'Star')
                    error('Input set is not an ImageStar or Star');
                end
                hs(i) = inputs(i).dev.h;
            end
            out = nnvhip_mex('affine_fc', obj.devW, hs);
            for i = n:-1:1
                if isa(inputs(i), 'ImageStar')
                    S(i) = nnvhip.ImageStar(nnvhip.DeviceSet(out(i)), 1, 1, obj.OutputSize);
                else
                    S(i) = nnvhip.Star(nnvhip.DeviceSet(out(i)));
                end
            end
        end
        function image = reach_star_single_input(obj, in_image)
            image = obj.reach_star_multipleInputs(in_image, 'single');
        end
        function delete(obj)
            if obj.devW ~= 0, nnvhip_mex('fc_destroy', obj.devW); end
        end
    end
end
