classdef (Abstract) RowMapLayer < handle
    % Shared plumbing of the layers that act row by row on the generator matrix (batch
    % normalisation, input normalisation): the per-row programme is built once per input shape and
    % kept on the device.  Subclasses return [ops; scopes] and the N x S operand matrix.
    %   ops:    0 add | 1 sub | 2 mul | 3 div        scopes: 0 centre column | 1 all columns
    properties (Transient)
        devMap = uint64(0);
        devKey = [];
    end
    methods (Abstract)
        [ops, scopes, params] = row_program(obj, h, w, c, isImage)
    end
    methods
        function S = apply_rowmap(obj, inputs)
            n = length(inputs);
            isImage = isa(inputs(1), 'ImageStar');
            if isImage
                key = [1 inputs(1).height inputs(1).width inputs(1).numChannel];
            else
                key = [0 inputs(1).dim 1 1];
            end
            if obj.devMap == 0 || ~isequal(key, obj.devKey)
                if obj.devMap ~= 0, nnvhip_mex('rowmap_destroy', obj.devMap); obj.devMap = uint64(0); end
                [ops, scopes, params] = obj.row_program(key(2), key(3), key(4), isImage);
                if isempty(ops)
                    S = inputs;          % the reference leaves the set unchanged
                    return;
                end
                obj.devMap = nnvhip_mex('rowmap_create', double(ops), double(scopes), double(params));
                obj.devKey = key;
            end
            hs = zeros(1, n, 'uint64');
            for i = 1:n, hs(i) = inputs(i).dev.h; end
            out = nnvhip_mex('affine_rowmap', obj.devMap, hs);
            for i = n:-1:1
                if isImage
                    S(i) = nnvhip.ImageStar(nnvhip.DeviceSet(out(i)), key(2), key(3), key(4));
                else
                    S(i) = nnvhip.Star(nnvhip.DeviceSet(out(i)));
                end
            end
        end
        function delete(obj)
            if obj.devMap ~= 0, nnvhip_mex('rowmap_destroy', obj.devMap); end
        end
    end
    methods (Static)
        function r = per_row(a, h, w, c)
            % scalar, per-channel (1 x 1 x c or vector) or full h x w x c values -> (h*w*c) x 1
            a = double(a);
            if isscalar(a)
                r = repmat(a, h*w*c, 1);
            elseif numel(a) == c
                r = repelem(a(:), h*w);
            elseif numel(a) == h*w*c
                r = a(:);
            else
                error('Inconsistent number of channels between scale array and the ImageStar');
            end
        end
    end
end
