classdef ImageStar < ImageStar
    % NNV ImageStar resident in HBM: the H x W x C x (numPred+1) tensor is the same device memory as
    % the (H*W*C) x (numPred+1) Star matrix (ImageStar.m:569-592, Star.m:1398-1418).
    % ImageStar is a handle class: the first read of V, C, d, pred_lb or pred_ub from outside the class fetches the
    % dense NNV array from the device and keeps it in the inherited field (subsref below); NNV methods that read
    % them from inside the class are overridden to fill the fields first (materialize()).
    properties
        dev = [];   % nnvhip.DeviceSet
    end
    methods
        function obj = ImageStar(varargin)
            % nnvhip.ImageStar(dev, h, w, c) | nnvhip.ImageStar(IS) | nnvhip.ImageStar(lb_im, ub_im)
            obj = obj@ImageStar();
            if nargin == 4
                obj.dev = varargin{1};
                obj.height = varargin{2}; obj.width = varargin{3}; obj.numChannel = varargin{4};
            elseif nargin == 1
                IS = varargin{1};
                S = nnvhip.Star(IS.toStar);
                obj.dev = S.dev;
                obj.height = IS.height; obj.width = IS.width; obj.numChannel = IS.numChannel;
                obj.im_lb = IS.im_lb; obj.im_ub = IS.im_ub;
            elseif nargin == 2
                lb = varargin{1}; ub = varargin{2}; n = size(lb);
                if numel(n) == 2, n(3) = 1; end
                S = nnvhip.Star(reshape(lb, [], 1), reshape(ub, [], 1));
                obj.dev = S.dev;
                obj.height = n(1); obj.width = n(2); obj.numChannel = n(3);
                obj.im_lb = lb; obj.im_ub = ub;
            end
            if ~isempty(obj.dev)
                dims = nnvhip_mex('star_dims', obj.dev.h);
                obj.numPred = dims(2);
            end
        end
        function S = toStar(obj)                     % ImageStar.m:569-592
            S = nnvhip.Star(obj.dev);
        end
        function [lb, ub] = estimateRanges(obj, varargin)   % ImageStar.m:836-885
            if isempty(obj.im_lb) || isempty(obj.im_ub)
                [l, u] = nnvhip_mex('estimate_ranges', obj.dev.h);
                obj.im_lb = reshape(l, obj.height, obj.width, obj.numChannel);
                obj.im_ub = reshape(u, obj.height, obj.width, obj.numChannel);
            end
            lb = obj.im_lb; ub = obj.im_ub;
        end
        function S = changeVarsPrecision(obj, precision)   % Star.m:1539-1560, ImageStar.m:673-695: the device store is fp64 only
            if ~strcmp(precision, 'double')
                error('this library keeps sets in double precision only');
            end
            S = obj;
        end
        function S = changeDevice(obj, deviceTarget)        % Star.m:1563-1585, ImageStar.m:697-720: the data is in HBM either way
            if ~any(strcmp(deviceTarget, {'cpu', 'gpu'}))
                error("Device target must be 'cpu' or 'gpu'.");
            end
            S = obj;
        end
        function materialize(obj)
            % fills the inherited dense fields from the device, once
            if isempty(obj.dev) || ~isempty(builtin('subsref', obj, substruct('.', 'V'))), return; end
            V = nnvhip_mex('fetch_V', obj.dev.h);
            obj.V = reshape(V, obj.height, obj.width, obj.numChannel, []);
            [obj.C, obj.d] = nnvhip_mex('fetch_constraints', obj.dev.h);
            [obj.pred_lb, obj.pred_ub] = nnvhip_mex('fetch_pred', obj.dev.h);
        end
        function varargout = subsref(obj, s)
            if isscalar(obj) && strcmp(s(1).type, '.') && any(strcmp(s(1).subs, {'V', 'C', 'd', 'pred_lb', 'pred_ub'}))
                obj.materialize();
            end
            [varargout{1:nargout}] = builtin('subsref', obj, s);
        end
        % ---- NNV methods that read the dense fields from inside the class ------------------------------------
        function varargout = getRanges(obj, varargin),  obj.materialize(); [varargout{1:nargout}] = getRanges@ImageStar(obj, varargin{:}); end
        function varargout = getRange(obj, varargin),   obj.materialize(); [varargout{1:nargout}] = getRange@ImageStar(obj, varargin{:}); end
        function varargout = estimateRange(obj, varargin), obj.materialize(); [varargout{1:nargout}] = estimateRange@ImageStar(obj, varargin{:}); end
        function bool = isEmptySet(obj),                 obj.materialize(); bool = isEmptySet@ImageStar(obj); end
        function bool = contains(obj, image),            obj.materialize(); bool = contains@ImageStar(obj, image); end
        function images = sample(obj, N),                obj.materialize(); images = sample@ImageStar(obj, N); end
        function image = evaluate(obj, pred_val),        obj.materialize(); image = evaluate@ImageStar(obj, pred_val); end
        function IS = affineMap(obj, scale, offset),     obj.materialize(); IS = affineMap@ImageStar(obj, scale, offset); end
        function IS = gather(obj)
            V = nnvhip_mex('fetch_V', obj.dev.h);
            [C, d] = nnvhip_mex('fetch_constraints', obj.dev.h);
            [plb, pub] = nnvhip_mex('fetch_pred', obj.dev.h);
            IS = ImageStar(reshape(V, obj.height, obj.width, obj.numChannel, []), C, d, plb, pub);
        end
    end
end
