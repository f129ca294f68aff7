classdef Star < Star
    % NNV Star whose [c V], predicate bounds and constraints live in HBM.
    % isa(S,'Star') stays true, so PosLin/NN guards (PosLin.m:902, NN.m:204-207) pass.
    % V, C, d stay empty on the host until gather() is called; dim/nVar are kept current.
    properties
        dev = [];   % nnvhip.DeviceSet
    end
    methods
        function obj = Star(varargin)
            % nnvhip.Star(S)       upload an existing NNV Star
            % nnvhip.Star(lb, ub)  Star(lb,ub) built on the device (Star.m:220-237)
            obj = obj@Star();
            if nargin == 1 && isa(varargin{1}, 'nnvhip.DeviceSet')
                obj.dev = varargin{1};
            elseif nargin == 1
                S = varargin{1};
                plb = S.predicate_lb; pub = S.predicate_ub;
                h = nnvhip_mex('star_create', double(S.V), double(S.C), double(S.d), double(plb), double(pub));
                obj.dev = nnvhip.DeviceSet(h);
                obj.state_lb = S.state_lb; obj.state_ub = S.state_ub;
            elseif nargin == 2
                h = nnvhip_mex('star_from_box', double(varargin{1}), double(varargin{2}));
                obj.dev = nnvhip.DeviceSet(h(1));
                obj.state_lb = varargin{1}; obj.state_ub = varargin{2};
            end
            if ~isempty(obj.dev)
                dims = nnvhip_mex('star_dims', obj.dev.h);
                obj.dim = dims(1); obj.nVar = dims(2);
            end
        end
        function S = affineMap(obj, W, b)            % Star.m:313-343
            if size(W, 2) ~= obj.dim
                error('Inconsistency between the affine mapping matrix and dimension of the star set');
            end
            L = nnvhip.FullyConnectedLayer(W, b);
            S = L.reach_star_single_input(obj);
        end
        function [lb, ub] = estimateRanges(obj)      % Star.m:1078-1106
            [lb, ub] = nnvhip_mex('estimate_ranges', obj.dev.h);
        end
        function IS = toImageStar(obj, h, w, c)      % Star.m:1398-1418 (a reshape: same device data)
            if obj.dim ~= h*w*c
                error('Inconsistent dimension in the ImageStar and the original Star set');
            end
            IS = nnvhip.ImageStar(obj.dev, h, w, c);
        end
        function S = changeVarsPrecision(obj, precision)   % Star.m:1539-1560: the device store is fp64 only
            if ~strcmp(precision, 'double')
                error('this library keeps sets in double precision only');
            end
            S = obj;
        end
        function S = changeDevice(obj, deviceTarget)        % Star.m:1563-1585: the data is in HBM either way
            if ~any(strcmp(deviceTarget, {'cpu', 'gpu'}))
                error("Device target must be 'cpu' or 'gpu'.");
            end
            S = obj;
        end
        function S = gather(obj)
            % plain NNV Star with dense host arrays, C/d in NNV's [C0;C1;C2;C3] layout
            V = nnvhip_mex('fetch_V', obj.dev.h);
            [C, d] = nnvhip_mex('fetch_constraints', obj.dev.h);
            [plb, pub] = nnvhip_mex('fetch_pred', obj.dev.h);
            S = Star(V, C, d, plb, pub);
        end
    end
end
