classdef Star < Star
    % NNV Star whose [c V], predicate bounds and constraints live in HBM.
    % isa(S,'Star') stays true, so PosLin/NN guards (PosLin.m:902, NN.m:204-207) pass.
    % dim/nVar are kept current.  The inherited fields V, C, d, predicate_lb, predicate_ub stay empty in the object;
    % a read of one of them from outside the class (S.V, S.C(1,:), ...) goes through subsref below, which fetches the
    % dense NNV array from the device (C, d in NNV's [C0;C1;C2;C3] layout, PosLin.m:711-735).  NNV methods that read
    % those fields from inside the class (a value class cannot intercept that) are overridden at the end of this
    % file: they gather() once and run NNV's own code on the plain Star.
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
            dims = nnvhip_mex('star_dims', obj.dev.h);
            if dims(5) ~= 0      % the outer zonotope of Star(lb,ub) and its affine images (Star.m:230-236, 332-340)
                S = Star(V, C, d, plb, pub, Zono(V(:, 1), V(:, 2:end)));
            else
                S = Star(V, C, d, plb, pub);
            end
            S.state_lb = obj.state_lb; S.state_ub = obj.state_ub;
        end
        function varargout = subsref(obj, s)
            % lazy property reads: S.V, S.C, S.d, S.predicate_lb, S.predicate_ub fetch from the device
            if isscalar(obj) && strcmp(s(1).type, '.') && ~isempty(obj.dev) && ...
                    any(strcmp(s(1).subs, {'V', 'C', 'd', 'predicate_lb', 'predicate_ub', 'Z'}))
                switch s(1).subs
                    case 'V', val = nnvhip_mex('fetch_V', obj.dev.h);
                    case 'C', [val, ~] = nnvhip_mex('fetch_constraints', obj.dev.h);
                    case 'd', [~, val] = nnvhip_mex('fetch_constraints', obj.dev.h);
                    case 'predicate_lb', [val, ~] = nnvhip_mex('fetch_pred', obj.dev.h);
                    case 'predicate_ub', [~, val] = nnvhip_mex('fetch_pred', obj.dev.h);
                    case 'Z'     % Star(lb,ub) and its affine images: Zono(c, gens) of the same set (Star.m:230-236, 332-340)
                        dims = nnvhip_mex('star_dims', obj.dev.h);
                        if dims(5) ~= 0
                            Vz = nnvhip_mex('fetch_V', obj.dev.h);
                            val = Zono(Vz(:, 1), Vz(:, 2:end));
                        else
                            val = [];
                        end
                end
                if numel(s) > 1
                    [varargout{1:nargout}] = subsref(val, s(2:end));
                else
                    varargout{1} = val;
                end
            else
                [varargout{1:nargout}] = builtin('subsref', obj, s);
            end
        end
        % ---- NNV methods that read V / C / d from inside the class: run on the gathered set ----------------
        function S = intersectHalfSpace(obj, H, g),   S = obj.gather().intersectHalfSpace(H, g); end      % Star.m:555-589
        function bool = isEmptySet(obj),              bool = obj.gather().isEmptySet(); end                % Star.m:1216-1232
        function [lb, ub] = getRanges(obj, varargin), [lb, ub] = obj.gather().getRanges(varargin{:}); end  % Star.m:973-990
        function B = getBox(obj),                     B = obj.gather().getBox(); end                       % Star.m:620-664
        function B = getBoxFast(obj),                 B = obj.gather().getBoxFast(); end
        function x = getMin(obj, varargin),           x = obj.gather().getMin(varargin{:}); end            % Star.m:710-745
        function x = getMax(obj, varargin),           x = obj.gather().getMax(varargin{:}); end
        function x = getMins(obj, varargin),          x = obj.gather().getMins(varargin{:}); end           % Star.m:784-870
        function x = getMaxs(obj, varargin),          x = obj.gather().getMaxs(varargin{:}); end
        function [lb, ub] = getRange(obj, varargin),  [lb, ub] = obj.gather().getRange(varargin{:}); end
        function bool = contains(obj, x),             bool = obj.gather().contains(x); end
        function bool = isSubSet(obj, S),             bool = obj.gather().isSubSet(S); end
        function V = sample(obj, N),                  V = obj.gather().sample(N); end
        function P = toPolyhedron(obj),               P = obj.gather().toPolyhedron(); end
        function Z = getZono(obj),                    Z = obj.gather().getZono(); end
        function S = MinkowskiSum(obj, X),            S = obj.gather().MinkowskiSum(X); end
        function S = resetRow(obj, map),              S = obj.gather().resetRow(map); end                  % Star.m:1442-1461
        function S = scalarMap(obj, a),               S = obj.gather().scalarMap(a); end
        function varargout = plot(obj, varargin),     [varargout{1:nargout}] = plot(obj.gather(), varargin{:}); end
    end
end
